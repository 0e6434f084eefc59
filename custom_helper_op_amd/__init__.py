"""MI355X-native plane-sweep cost-volume operator (drop-in for the cost-volume ops of
zhuimeng999/custom_helper_op).  The public names follow custom_helper_op/__init__.py."""
from .layers import CostMapLayer, CostMapLayerV2
from .ops import (InvalidArgumentError, combine_projection, cost_aggregate, cost_aggregate_grad,
                  cost_aggregate_filled, cost_aggregate_raw, cost_default_fill, cost_volume, cost_volume_grad,
                  cost_volume_grad_v2, cost_volume_grad_v3, cost_volume_raw, cost_volume_v2,
                  cost_volume_v2_filled, cost_volume_v2_raw, cost_volume_v3, cost_volume_v3_raw, feature_aggregate,
                  feature_aggregate_grad, feature_aggregate_raw, sample_coords)

__all__ = ["cost_volume", "cost_volume_v2", "cost_volume_v3", "cost_aggregate", "feature_aggregate",
           "cost_volume_grad", "cost_volume_grad_v2", "cost_volume_grad_v3", "cost_aggregate_grad",
           "feature_aggregate_grad", "cost_volume_raw", "cost_volume_v2_raw", "cost_volume_v3_raw",
           "cost_aggregate_raw", "feature_aggregate_raw", "cost_default_fill", "combine_projection",
           "cost_aggregate_filled", "cost_volume_v2_filled",
           "CostMapLayer", "CostMapLayerV2", "sample_coords", "InvalidArgumentError"]
