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
 *   custom_helper_op/cc/kernels/cost_volume_kernels_gpu_v3.cu.cc
 *       :33-143  CostMeanVolumeV3Kernel      -> chop_oracle_cost_volume_v3_fwd_* (reduce 0)
 *       :145-261 CostMinVolumeV3Kernel       -> chop_oracle_cost_volume_v3_fwd_* (reduce 1)
 *       :376-517 CostMeanVolumeGradV3Kernel  -> chop_oracle_cost_volume_v3_bwd_* (reduce 0)
 *       :519-639 CostMinVolumeGradV3Kernel   -> chop_oracle_cost_volume_v3_bwd_* (reduce 1)
 *   custom_helper_op/cc/kernels/feature_aggregate_kernels_gpu.cu.cc
 *       :33-121  FeatureAggregateKernel      -> chop_oracle_feature_aggregate_fwd_*
 *       :219-326 FeatureAggregateGradKernel  -> chop_oracle_feature_aggregate_bwd_*
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
 *   CostVolumeV3 forward: pinned by the composite (all group pairs by einsum, maximum and
 *     arg-maximum), by brute force including all-negative correlations (the seed survives)
 *     and exact ties (first pair wins), and by the pinned V2 oracle for one group.
 *     Backward: by the V2 gradient for one group and by finite differences in float64.
 *     Where the reference reads out of bounds (no pair above the seed, :495-496) the view
 *     contributes nothing here; that choice is not a parity claim.
 *   FeatureAggregate forward: pinned by the composite (also with a source size different
 *     from the output grid) and, bit for bit, by the pinned V2 oracle against a reference
 *     image of ones with one channel per group.  Backward: by that V2 gradient and by
 *     finite differences.
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
