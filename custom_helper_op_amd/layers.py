"""The reference's cost-map layers on top of the operators
(custom_helper_op/python/layers/custom_layers.py:33-84), as torch modules.

``CostMapLayer`` runs CostAggregate and ``CostMapLayerV2`` runs CostVolumeV2; both replace the
cost of every voxel that no source view covered by a scalar ``default_cost`` -- here inside
the op's own store, so the forward is one kernel.
``default_type`` keeps the reference's meaning: ``'DYNAMIC'`` a trainable scalar initialised to
zero, ``'CONSTANT'`` the same scalar but frozen, a tensor (V2) or number the fixed value itself.
"""
import torch

from . import ops


class _CostMapBase(torch.nn.Module):
    def __init__(self, reduce_method, half_centor, default_type):
        super().__init__()
        if reduce_method not in ("MEAN", "MIN"):
            raise ops.InvalidArgumentError("reduce_method must be MEAN or MIN")
        self.reduce_method = reduce_method
        self.half_centor = half_centor
        if isinstance(default_type, str):
            if default_type not in ("CONSTANT", "DYNAMIC"):
                raise ops.InvalidArgumentError("default_type must be CONSTANT, DYNAMIC or a value")
            self.default_cost = torch.nn.Parameter(torch.zeros(()),
                                                   requires_grad=default_type == "DYNAMIC")
        else:
            self.register_buffer("default_cost", torch.as_tensor(default_type, dtype=torch.float32))

    def _default(self, like, real_dtype):
        return self.default_cost.to(device=like.device, dtype=real_dtype)


class CostMapLayer(_CostMapBase):
    """``(ref_image, src_images, base_plane, offsets, Rs, Ts) -> (cost [B,H,W,D], cost_mask)``
    (custom_layers.py:33-57)."""

    def __init__(self, reduce_method="MIN", half_centor=True, default_type="DYNAMIC"):
        super().__init__(reduce_method, half_centor, default_type)

    def forward(self, inputs):
        ref = inputs[0]
        return ops.cost_aggregate_filled(*inputs, self._default(ref, ref.dtype),
                                         reduce_method=self.reduce_method,
                                         half_centor=self.half_centor)


class CostMapLayerV2(_CostMapBase):
    """``(ref_image, src_images, depth_grid, Rs, Ts) -> (cost [B,H,W,D,groups], cost_mask)``
    (custom_layers.py:59-84)."""

    def __init__(self, reduce_method="MIN", half_centor=True, default_type="DYNAMIC", groups=1):
        super().__init__(reduce_method, half_centor, default_type)
        self.groups = groups

    def forward(self, inputs):
        ref = inputs[0]
        real = torch.float32 if ref.dtype in (torch.float16, torch.bfloat16) else ref.dtype
        return ops.cost_volume_v2_filled(*inputs, self._default(ref, real),
                                         reduce_method=self.reduce_method, groups=self.groups,
                                         half_centor=self.half_centor)
