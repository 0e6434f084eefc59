/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the reference's plane-sweep cost-volume kernels
 * (zhuimeng999/custom_helper_op).  It exists to check the HIP library and to time a
 * CPU baseline; only the test-suite, the smoke check and the benchmark's cpu_baseline
 * leg may load it.  The HIP library never links, loads or calls anything in here.
 *
 * Followed source (paths relative to the reference checkout):
 *   custom_helper_op/cc/kernels/cost_volume_kernels_gpu.cu.cc
 *       :33-131  CostMeanVolumeKernel        -> chop_oracle_cost_volume_fwd_*  (reduce 0)
 *       :133-228 CostMinVolumeKernel         -> chop_oracle_cost_volume_fwd_*  (reduce 1)
 *       :342-456 CostMeanVolumeGradKernel    -> chop_oracle_cost_volume_bwd_*  (reduce 0)
 *       :458-577 CostMinVolumeGradKernel     -> chop_oracle_cost_volume_bwd_*  (reduce 1)
 *       :637-642 SetZeroBig launches         -> memset of the three gradients
 *   custom_helper_op/cc/kernels/cost_volume_kernels_gpu_v2.cu.cc
 *       :33-135  CostMeanVolumeV2Kernel      -> chop_oracle_cost_volume_v2_fwd_* (reduce 0)
 *       :137-235 CostMinVolumeV2Kernel       -> chop_oracle_cost_volume_v2_fwd_* (reduce 1)
 *       :349-479 CostMeanVolumeGradV2Kernel  -> chop_oracle_cost_volume_v2_bwd_* (reduce 0)
 *       :481-601 CostMinVolumeGradV2Kernel   -> chop_oracle_cost_volume_v2_bwd_* (reduce 1)
 *
 *   custom_helper_op/cc/kernels/cost_aggregate_kernels_gpu.cu.cc
 *       :33-126  CostMeanAggregateKernel     -> chop_oracle_cost_aggregate_fwd_* (reduce 0)
 *       :128-229 CostMinAggregateKernel      -> chop_oracle_cost_aggregate_fwd_* (reduce 1)
 *       :338-452 CostMeanAggregateGradKernel -> chop_oracle_cost_aggregate_bwd_* (reduce 0)
 *       :454-563 CostMinAggregateGradKernel  -> chop_oracle_cost_aggregate_bwd_* (reduce 1)
 *
 * Parity status of each function (what pins it is in tests/test_oracle_*.py):
 *   forward MEAN/MIN (V1), MEAN/MAX (V2): pinned by an independent float64 composite that
 *     restates the reference tests' own oracle, by closed-form camera cases, by a
 *     brute-force Python loop on tiny inputs, and by invariants.
 *   backward, all four: pinned by central finite differences of the forward in float64
 *     with the reference tests' loss and tolerance, and by conservation identities.
 *   aggregate forward MEAN: pinned against the pinned cost-volume forward (it is its mean
 *     over channels) and by the composite; MIN: by the composite and brute force.
 *   aggregate backward: MEAN pinned against the pinned cost-volume backward fed the
 *     upstream gradient broadcast over channels and divided by C; both reduces by finite
 *     differences in float64.
 *   sample_coords: pinned by the float64 composite's coordinates.
 *   NOT pinned: the rounding of a CUDA build of the reference (nvcc contracts a*b+c into
 *     fused multiply-adds and the reference is built with ftz=true).  No such build or
 *     output of one exists here, so the canonical fp32 rounding is defined as "literal
 *     source order, no contraction, IEEE denormals"; bit-exactness claims are relative
 *     to that definition -- "parity unpinned" for the nvcc rounding pattern only.
 *
 * threads: 1 reproduces the sequential voxel order exactly; >1 splits pixels into
 * contiguous ranges (OpenMP) -- forward results are identical, backward results differ
 * only in the order src_grad contributions from different ranges are summed.
 *
 * Status codes: 0 ok, 2 bad dims, 3 bad reduce, 4 bad groups, 8 out of memory.
 */
#include <float.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define REAL float
#define SFX f32
#define REAL_MAX FLT_MAX
#define REAL_MINPOS FLT_MIN
#include "costvol_oracle_body.inc"
#undef REAL
#undef SFX
#undef REAL_MAX
#undef REAL_MINPOS

#define REAL double
#define SFX f64
#define REAL_MAX DBL_MAX
#define REAL_MINPOS DBL_MIN
#include "costvol_oracle_body.inc"
#undef REAL
#undef SFX
#undef REAL_MAX
#undef REAL_MINPOS

int chop_oracle_abi_version(void) { return 1; }
