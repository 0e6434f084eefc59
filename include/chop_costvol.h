/*
 * libchop_costvol -- plane-sweep cost-volume operator for AMD MI355X (gfx950), C ABI.
 *
 * Drop-in replacement for the device functors of zhuimeng999/custom_helper_op's
 * CostVolume / CostVolumeGrad / CostVolumeV2 / CostVolumeGradV2 ops.  Every entry
 * point takes plain device pointers and sizes, enqueues work on the given HIP stream
 * and returns immediately; it never synchronises and never allocates or frees device
 * memory.  The caller owns every buffer.  Gradient outputs may arrive uninitialised:
 * the library clears what it accumulates into.
 *
 * Tensor layouts (dense, row-major, innermost last), as registered by the reference
 * (custom_helper_op/cc/ops/custom_helper_ops.cc:190-307):
 *   ref        [B,H,W,C]            src        [B,N,srcH,srcW,C]
 *   base_plane [B,H,W,1]            offsets    [B,D]            (V1 depth = base + offset)
 *   depth_grid [B,H,W,D]                                          (V2 depth)
 *   Rs         [B,N,3,3]  = K_src R K_ref^-1        Ts [B,N,3] = K_src t
 *   cost       [B,H,W,D,C] (V1)  /  [B,H,W,D,groups] (V2)
 *   mask int32 [B,H,W,D,1] for CHOP_REDUCE_MEAN (valid-view count)
 *              [B,H,W,D,C|groups] for CHOP_REDUCE_MIN (winning view or -1)
 *   gradients shaped like ref, src, base_plane (V1) / depth_grid (V2).
 *
 * Return value: 0 on success, a chop_status otherwise; chop_last_error_string()
 * describes the last failure on the calling thread.  Zero-sized work is a successful
 * no-op (the reference aborts on it, cost_volume_kernels_gpu.cu.cc:238).
 * All entry points are re-entrant and may be called from several host threads.
 */
#ifndef CHOP_COSTVOL_H_
#define CHOP_COSTVOL_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum chop_status {
  CHOP_OK = 0,
  CHOP_ERR_NULL_POINTER = 1,   /* a required buffer is NULL */
  CHOP_ERR_BAD_DIMS = 2,       /* negative or overflowing dimension */
  CHOP_ERR_BAD_ENUM = 3,       /* reduce is neither CHOP_REDUCE_MEAN nor CHOP_REDUCE_MIN */
  CHOP_ERR_BAD_GROUPS = 4,     /* groups <= 0 or C % groups != 0 */
  CHOP_ERR_LAUNCH = 5,         /* HIP reported an error when the work was enqueued */
  CHOP_ERR_WORKSPACE = 6,      /* workspace NULL, misaligned or too small */
  CHOP_ERR_NO_DEVICE = 7       /* no usable HIP device */
} chop_status;

/* reduce_method attr of the ops: "MEAN" / "MIN"
 * (reference enum COST_REDUCE_METHOD, custom_helper_op/cc/kernels/cost_volume.h:35). */
enum { CHOP_REDUCE_MEAN = 0, CHOP_REDUCE_MIN = 1 };

/* Element types of the 16-bit storage extension. */
enum { CHOP_STORAGE_F16 = 1, CHOP_STORAGE_BF16 = 2 };

int chop_abi_version(void);
/* Optional set-up for the current device, outside any stream capture: locates the static
 * scratch array of chop_cost_volume_bwd_16_static on this device (one runtime query, cached
 * per device).  Every other entry point works without it; chop_cost_volume_bwd_16_static
 * makes the same query on its first call on a device, unless that call is being captured
 * into a HIP graph, in which case it returns CHOP_ERR_WORKSPACE and asks for this call.
 * Returns CHOP_ERR_NO_DEVICE when there is no usable device.  No counterpart in the
 * reference (its functors keep no state). */
int chop_init(void);
const char *chop_last_error_string(void);

/* ---- CostVolume forward ------------------------------------------------------------
 * Replaces functor::CostVolumeFunctor<GPUDevice,T,half_centor>::operator()
 * (declared custom_helper_op/cc/kernels/cost_volume.h:37-80, defined
 * cost_volume_kernels_gpu.cu.cc:289-335, called from CostVolumeOp::Compute,
 * cost_volume_kernels.cc:128-136).  `stream` is a hipStream_t. */
int chop_cost_volume_fwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                             int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                             int64_t srcW, const float *ref, const float *src,
                             const float *base_plane, const float *offsets, const float *Rs,
                             const float *Ts, float *cost, int32_t *mask);
int chop_cost_volume_fwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                             int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                             int64_t srcW, const double *ref, const double *src,
                             const double *base_plane, const double *offsets, const double *Rs,
                             const double *Ts, double *cost, int32_t *mask);

/* ---- CostVolume backward -----------------------------------------------------------
 * Replaces functor::CostVolumeGradFunctor<GPUDevice,T,half_centor>::operator()
 * (cost_volume.h:82-133, cost_volume_kernels_gpu.cu.cc:590-655, called from
 * CostVolumeGradOp::Compute, cost_volume_kernels.cc:263-271), including the three
 * SetZeroBig launches (:637-642).
 *
 * In the CostVolume, CostVolumeV2 and CostAggregate backward entry points the third
 * gradient (base_plane_grad / depth_grid_grad) may be NULL: it is then neither cleared
 * nor computed, the other two gradients are unchanged.  The reference always computes
 * it; a caller whose depth hypotheses are constants saves the work. */
int chop_cost_volume_bwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                             int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                             int64_t srcW, const float *ref, const float *src,
                             const float *base_plane, const float *offsets, const float *Rs,
                             const float *Ts, const float *cost_grad, const int32_t *mask,
                             float *ref_grad, float *src_grad, float *base_plane_grad);
int chop_cost_volume_bwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                             int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                             int64_t srcW, const double *ref, const double *src,
                             const double *base_plane, const double *offsets, const double *Rs,
                             const double *Ts, const double *cost_grad, const int32_t *mask,
                             double *ref_grad, double *src_grad, double *base_plane_grad);

/* ---- CostVolumeV2 forward / backward ------------------------------------------------
 * Replace functor::CostVolumeV2Functor / CostVolumeGradV2Functor
 * (custom_helper_op/cc/kernels/cost_volume_v2.h:37-133,
 * cost_volume_kernels_gpu_v2.cu.cc:296-342 and :614-680, called from
 * cost_volume_kernels_v2.cc:130-138 and :265-273).  The third gradient is the
 * depth_grid gradient (registered under the name base_plane_grad,
 * custom_helper_ops.cc:301); voxels skipped by the mask receive 0. */
int chop_cost_volume_v2_fwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const float *ref, const float *src,
                                const float *depth_grid, const float *Rs, const float *Ts,
                                float *cost, int32_t *mask);
int chop_cost_volume_v2_fwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const double *ref, const double *src,
                                const double *depth_grid, const double *Rs, const double *Ts,
                                double *cost, int32_t *mask);
int chop_cost_volume_v2_bwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const float *ref, const float *src,
                                const float *depth_grid, const float *Rs, const float *Ts,
                                const float *cost_grad, const int32_t *mask, float *ref_grad,
                                float *src_grad, float *depth_grid_grad);
int chop_cost_volume_v2_bwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const double *ref, const double *src,
                                const double *depth_grid, const double *Rs, const double *Ts,
                                const double *cost_grad, const int32_t *mask, double *ref_grad,
                                double *src_grad, double *depth_grid_grad);

/* ---- CostAggregate forward / backward -----------------------------------------------
 * The squared differences of all channels summed into one value per voxel.
 * Replaces functor::CostAggregateFunctor<GPUDevice,T,half_centor>::operator() and
 * functor::CostAggregateGradFunctor<GPUDevice,T,half_centor>::operator()
 * (declared custom_helper_op/cc/kernels/cost_aggregate.h:38-133, defined
 * cost_aggregate_kernels_gpu.cu.cc:290-331 and :586-646, called from
 * CostAggregateOp::Compute and CostAggregateGradOp::Compute,
 * cost_aggregate_kernels.cc:120-128 and :247-255).
 * cost is [B,H,W,D]; mask is int32 [B,H,W,D]: the number of accepted views (MEAN) or the
 * view with the smallest sum, -1 if none was accepted (MIN).  MEAN divides the sum by
 * (accepted views * C), MIN by C; a voxel no view accepted gets cost 0.
 * The backward takes cost_grad [B,H,W,D] and the forward's mask. */
int chop_cost_aggregate_fwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, const float *ref, const float *src,
                                const float *base_plane, const float *offsets, const float *Rs,
                                const float *Ts, float *cost, int32_t *mask);
int chop_cost_aggregate_fwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, const double *ref, const double *src,
                                const double *base_plane, const double *offsets,
                                const double *Rs, const double *Ts, double *cost, int32_t *mask);
int chop_cost_aggregate_bwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, const float *ref, const float *src,
                                const float *base_plane, const float *offsets, const float *Rs,
                                const float *Ts, const float *cost_grad, const int32_t *mask,
                                float *ref_grad, float *src_grad, float *base_plane_grad);
int chop_cost_aggregate_bwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, const double *ref, const double *src,
                                const double *base_plane, const double *offsets,
                                const double *Rs, const double *Ts, const double *cost_grad,
                                const int32_t *mask, double *ref_grad, double *src_grad,
                                double *base_plane_grad);

/* ---- CostVolumeV3 forward / backward -------------------------------------------------
 * Per accepted view, the largest dot product between any channel group of the bilinear
 * source sample and any channel group of the reference pixel (groups x groups pairs of
 * C/groups channels each, at most 8 channels per group); one value per voxel.
 * Replaces functor::CostVolumeV3Functor<GPUDevice,T,half_centor>::operator() and
 * functor::CostVolumeGradV3Functor<GPUDevice,T,half_centor>::operator()
 * (declared custom_helper_op/cc/kernels/cost_volume_v3.h:40-141, defined
 * cost_volume_kernels_gpu_v3.cu.cc:323-369 and :653-719, called from
 * CostVolumeV3Op::Compute and CostVolumeGradV3Op::Compute,
 * cost_volume_kernels_v3.cc:137-145 and :274-282).
 * cost is [B,H,W,D,1].  MEAN: mask int32 [B,H,W,D,1] = number of accepted views, cost =
 * mean of the views' maxima (each seeded with the smallest positive normal number, as the
 * reference does), 0 where no view was accepted.  MIN: cost = the largest value over all
 * views and pairs, mask int32 [B,H,W,D,3] = (view, reference group, source group) of the
 * winner, all -1 and cost 0 when nothing exceeded the seed.
 * The backward takes cost_grad [B,H,W,D,1] and the forward's mask.  A view whose best
 * pair does not exceed the seed contributes no gradient (the reference indexes channel
 * group -1 there, cost_volume_kernels_gpu_v3.cu.cc:495-496).
 * Extra status: CHOP_ERR_BAD_GROUPS when groups does not divide C or C/groups > 8
 * (cost_volume_kernels_v3.cc:111-115). */
int chop_cost_volume_v3_fwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const float *ref, const float *src,
                                const float *base_plane, const float *offsets, const float *Rs,
                                const float *Ts, float *cost, int32_t *mask);
int chop_cost_volume_v3_fwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const double *ref, const double *src,
                                const double *base_plane, const double *offsets,
                                const double *Rs, const double *Ts, double *cost, int32_t *mask);
int chop_cost_volume_v3_bwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const float *ref, const float *src,
                                const float *base_plane, const float *offsets, const float *Rs,
                                const float *Ts, const float *cost_grad, const int32_t *mask,
                                float *ref_grad, float *src_grad, float *base_plane_grad);
int chop_cost_volume_v3_bwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const double *ref, const double *src,
                                const double *base_plane, const double *offsets,
                                const double *Rs, const double *Ts, const double *cost_grad,
                                const int32_t *mask, double *ref_grad, double *src_grad,
                                double *base_plane_grad);

/* ---- FeatureAggregate forward / backward ---------------------------------------------
 * The warp alone: mapped_feature [B,H,W,D,N,C] holds the bilinear sample of every source
 * view at every voxel (zeros where the view is not accepted) and mapped_mask int32
 * [B,H,W,D,N,1] is 1 / 0.  H and W are those of base_plane [B,H,W,1]; the source images
 * [B,N,srcH,srcW,C] may have another size.
 * Replaces functor::FeatureAggregateFunctor<GPUDevice,T,half_centor>::operator() and
 * functor::FeatureAggregateGradFunctor<GPUDevice,T,half_centor>::operator()
 * (declared custom_helper_op/cc/kernels/feature_aggregate.h:36-128, defined
 * feature_aggregate_kernels_gpu.cu.cc:182-213 and :339-388, called from
 * FeatureAggregateOp::Compute and FeatureAggregateGradOp::Compute,
 * feature_aggregate_kernels.cc:105-113 and :223-231).
 * The backward takes mapped_feature_grad [B,H,W,D,N,C] and the forward's mask and writes
 * src_grad [B,N,srcH,srcW,C] and base_plane_grad [B,H,W,1]. */
int chop_feature_aggregate_fwd_f32(void *stream, int half_centor, int64_t B, int64_t H, int64_t W,
                                   int64_t C, int64_t D, int64_t N, int64_t srcH, int64_t srcW,
                                   const float *src, const float *base_plane,
                                   const float *offsets, const float *Rs, const float *Ts,
                                   float *mapped_feature, int32_t *mapped_mask);
int chop_feature_aggregate_fwd_f64(void *stream, int half_centor, int64_t B, int64_t H, int64_t W,
                                   int64_t C, int64_t D, int64_t N, int64_t srcH, int64_t srcW,
                                   const double *src, const double *base_plane,
                                   const double *offsets, const double *Rs, const double *Ts,
                                   double *mapped_feature, int32_t *mapped_mask);
int chop_feature_aggregate_bwd_f32(void *stream, int half_centor, int64_t B, int64_t H, int64_t W,
                                   int64_t C, int64_t D, int64_t N, int64_t srcH, int64_t srcW,
                                   const float *src, const float *base_plane,
                                   const float *offsets, const float *Rs, const float *Ts,
                                   const float *mapped_feature_grad, const int32_t *mapped_mask,
                                   float *src_grad, float *base_plane_grad);
int chop_feature_aggregate_bwd_f64(void *stream, int half_centor, int64_t B, int64_t H, int64_t W,
                                   int64_t C, int64_t D, int64_t N, int64_t srcH, int64_t srcW,
                                   const double *src, const double *base_plane,
                                   const double *offsets, const double *Rs, const double *Ts,
                                   const double *mapped_feature_grad,
                                   const int32_t *mapped_mask, double *src_grad,
                                   double *base_plane_grad);

/* ---- callers on either side of the ops ----------------------------------------------
 * Default fill: what CostMapLayer / CostMapLayerV2 do with the op's outputs,
 *   out = where(valid(mask), cost, *default_cost),  valid = mask > 0 (MEAN) or mask >= 0 (MIN)
 * (custom_helper_op/python/layers/custom_layers.py:52-57 and :78-83; `default_cost` is the
 * layer's scalar weight and lives in device memory).  cost and out hold mask_count * inner
 * elements, `inner` consecutive ones per mask entry (CostAggregate: inner 1, mask [B,H,W,D];
 * CostVolumeV2 MEAN: inner = groups, mask [B,H,W,D,1]; CostVolumeV2 MIN: inner 1, mask
 * [B,H,W,D,groups]).  out may be the cost buffer itself.
 * The gradient of that `where`: cost_grad = out_grad where valid and 0 elsewhere (cost_grad
 * may be NULL when only the scalar's gradient is wanted),
 * *default_grad = sum of out_grad where not valid (the entry zeroes it first). */
int chop_cost_default_fill_f32(void *stream, int reduce, int64_t mask_count, int64_t inner,
                               const float *cost, const int32_t *mask, const float *default_cost,
                               float *out);
int chop_cost_default_fill_f64(void *stream, int reduce, int64_t mask_count, int64_t inner,
                               const double *cost, const int32_t *mask,
                               const double *default_cost, double *out);
int chop_cost_default_fill_grad_f32(void *stream, int reduce, int64_t mask_count, int64_t inner,
                                    const float *out_grad, const int32_t *mask, float *cost_grad,
                                    float *default_grad);
int chop_cost_default_fill_grad_f64(void *stream, int reduce, int64_t mask_count, int64_t inner,
                                    const double *out_grad, const int32_t *mask,
                                    double *cost_grad, double *default_grad);
/* combine_projection (custom_helper_op/python/ops/op_tests/cost_volume_op_test.py:115-134;
 * the same helper is repeated in the other op tests): the Rs [B,N,3,3] and Ts [B,N,3] the ops
 * take, from ref_cam [B,2,4,4] and src_cam [B,N,2,4,4] (first 4x4 the extrinsic [R|t], second
 * the intrinsic K in its upper-left 3x3) and scale [3] (multiplies the rows of both K; then
 * 0.5 is added to both principal points):
 *   R = src_K (src_R ref_R^T) ref_K^-1,   T = src_K (src_t - src_R ref_R^T ref_t). */
/* The same for an upstream gradient in 16-bit storage (CHOP_STORAGE_F16 / _BF16), as the
 * 16-bit CostVolumeV2 layer produces it: read as stored, summed in float; cost_grad (same
 * storage type, may be NULL) as above. */
int chop_cost_default_fill_grad_16(void *stream, int storage, int reduce, int64_t mask_count,
                                   int64_t inner, const void *out_grad, const int32_t *mask,
                                   void *cost_grad, float *default_grad);
int chop_combine_projection_f32(void *stream, int64_t B, int64_t N, const float *ref_cam,
                                const float *src_cam, const float *scale, float *Rs, float *Ts);
int chop_combine_projection_f64(void *stream, int64_t B, int64_t N, const double *ref_cam,
                                const double *src_cam, const double *scale, double *Rs,
                                double *Ts);

/* The two layers' forward as one call: CostAggregate (CostMapLayer,
 * custom_layers.py:51-57) and CostVolumeV2 (CostMapLayerV2, :77-83) with that default fill
 * folded into the kernels' store, so the cost volume is written once instead of being read
 * back and rewritten.  `default_cost` is the layer's device scalar; cost and mask are what
 * chop_cost_aggregate_fwd_* / chop_cost_volume_v2_fwd_* followed by chop_cost_default_fill_*
 * produce, bit for bit.  The gradients are those of the plain ops (voxels that received the
 * default take no gradient there either) plus chop_cost_default_fill_grad_* for the scalar. */
int chop_cost_aggregate_fwd_fill_f32(void *stream, int reduce, int half_centor, int64_t B,
                                     int64_t H, int64_t W, int64_t C, int64_t D, int64_t N,
                                     int64_t srcH, int64_t srcW, const float *ref,
                                     const float *src, const float *base_plane,
                                     const float *offsets, const float *Rs, const float *Ts,
                                     const float *default_cost, float *cost, int32_t *mask);
int chop_cost_aggregate_fwd_fill_f64(void *stream, int reduce, int half_centor, int64_t B,
                                     int64_t H, int64_t W, int64_t C, int64_t D, int64_t N,
                                     int64_t srcH, int64_t srcW, const double *ref,
                                     const double *src, const double *base_plane,
                                     const double *offsets, const double *Rs, const double *Ts,
                                     const double *default_cost, double *cost, int32_t *mask);
int chop_cost_volume_v2_fwd_fill_f32(void *stream, int reduce, int half_centor, int64_t B,
                                     int64_t H, int64_t W, int64_t C, int64_t D, int64_t N,
                                     int64_t srcH, int64_t srcW, int groups, const float *ref,
                                     const float *src, const float *depth_grid, const float *Rs,
                                     const float *Ts, const float *default_cost, float *cost,
                                     int32_t *mask);
int chop_cost_volume_v2_fwd_fill_f64(void *stream, int reduce, int half_centor, int64_t B,
                                     int64_t H, int64_t W, int64_t C, int64_t D, int64_t N,
                                     int64_t srcH, int64_t srcW, int groups, const double *ref,
                                     const double *src, const double *depth_grid,
                                     const double *Rs, const double *Ts,
                                     const double *default_cost, double *cost, int32_t *mask);

/* ---- 16-bit storage extension --------------------------------------------------------
 * No counterpart in the reference, whose ops register float32 and float64 only
 * (custom_helper_ops.cc:197,234).  ref, src, cost, cost_grad, ref_grad and src_grad
 * hold IEEE half (CHOP_STORAGE_F16) or bfloat16 (CHOP_STORAGE_BF16) elements; depth
 * inputs, camera matrices and depth gradients stay float; coordinates and all
 * arithmetic are fp32, identical to the f32 entry points run on the widened inputs.
 * `depth_grid` non-NULL selects per-pixel hypotheses for the V1 squared-difference
 * reduce (base_plane/offsets are then ignored and the third gradient has the shape of
 * depth_grid).
 * With CHOP_REDUCE_MIN an element no view reached keeps the fp32 seed rounded to the storage
 * type: the largest float becomes +infinity in both 16-bit types, the group correlation's
 * smallest normal float stays what it is in bfloat16 and becomes 0 in half; the mask entry
 * (-1) marks such an element, as in the float ops.
 * The backward accumulates source/reference gradients in fp32 inside `workspace`
 * (device memory, 256-byte aligned, at least chop_cost_volume_bwd16_workspace_bytes). */
size_t chop_cost_volume_bwd16_workspace_bytes(int64_t B, int64_t H, int64_t W, int64_t C,
                                              int64_t N, int64_t srcH, int64_t srcW);
int chop_cost_volume_fwd_16(void *stream, int storage, int reduce, int half_centor, int64_t B,
                            int64_t H, int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                            int64_t srcW, const void *ref, const void *src,
                            const float *base_plane, const float *offsets,
                            const float *depth_grid, const float *Rs, const float *Ts,
                            void *cost, int32_t *mask);
int chop_cost_volume_bwd_16(void *stream, int storage, int reduce, int half_centor, int64_t B,
                            int64_t H, int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                            int64_t srcW, const void *ref, const void *src,
                            const float *base_plane, const float *offsets,
                            const float *depth_grid, const float *Rs, const float *Ts,
                            const void *cost_grad, const int32_t *mask, void *ref_grad,
                            void *src_grad, float *depth_grad, void *workspace,
                            size_t workspace_bytes);
/* chop_cost_volume_bwd_16 for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in
 * the reference.  Same arguments and results as chop_cost_volume_bwd_16 without the
 * workspace: the fp32 gradient images live in a static device array of
 * chop_static_scratch_bytes() (32 MiB) that every GPU the library runs on holds until the
 * process ends; a shape whose chop_cost_volume_bwd16_workspace_bytes exceeds that is
 * rejected with CHOP_ERR_WORKSPACE.  The call allocates and frees nothing.  All calls on one
 * GPU share the array: calls that overlap in time on the same GPU (different streams or
 * host threads) race and must be serialised by the caller.  A caller that captures the call
 * into a HIP graph calls chop_init() (or this entry point) once on the device beforehand. */
size_t chop_static_scratch_bytes(void);
int chop_cost_volume_bwd_16_static(void *stream, int storage, int reduce, int half_centor,
                                   int64_t B, int64_t H, int64_t W, int64_t C, int64_t D,
                                   int64_t N, int64_t srcH, int64_t srcW, const void *ref,
                                   const void *src, const float *base_plane,
                                   const float *offsets, const float *depth_grid,
                                   const float *Rs, const float *Ts, const void *cost_grad,
                                   const int32_t *mask, void *ref_grad, void *src_grad,
                                   float *depth_grad);
int chop_cost_volume_v2_fwd_16(void *stream, int storage, int reduce, int half_centor, int64_t B,
                               int64_t H, int64_t W, int64_t C, int64_t D, int64_t N,
                               int64_t srcH, int64_t srcW, int groups, const void *ref,
                               const void *src, const float *depth_grid, const float *Rs,
                               const float *Ts, void *cost, int32_t *mask);
int chop_cost_volume_v2_fwd_fill_16(void *stream, int storage, int reduce, int half_centor,
                                    int64_t B, int64_t H, int64_t W, int64_t C, int64_t D,
                                    int64_t N, int64_t srcH, int64_t srcW, int groups,
                                    const void *ref, const void *src, const float *depth_grid,
                                    const float *Rs, const float *Ts, const float *default_cost,
                                    void *cost, int32_t *mask);
int chop_cost_volume_v2_bwd_16(void *stream, int storage, int reduce, int half_centor, int64_t B,
                               int64_t H, int64_t W, int64_t C, int64_t D, int64_t N,
                               int64_t srcH, int64_t srcW, int groups, const void *ref,
                               const void *src, const float *depth_grid, const float *Rs,
                               const float *Ts, const void *cost_grad, const int32_t *mask,
                               void *ref_grad, void *src_grad, float *depth_grid_grad,
                               void *workspace, size_t workspace_bytes);

/* ---- diagnostics ------------------------------------------------------------------------
 * No counterpart in the reference.  Writes, for every (voxel, view), the source-view
 * sample coordinate exactly as the kernels above compute it, so that coordinates,
 * truncated indices and acceptance can be compared bit for bit with another
 * implementation.  Outputs are [B,H,W,D,N]: sw/sh the coordinates (0 when the point is
 * behind the camera), fh/fw the truncated indices (-1 unless accepted), state 0 behind
 * the camera, 1 outside the open rectangle (0,srcW-1)x(0,srcH-1), 2 accepted.
 * depth_grid non-NULL selects the V2 depth source. */
int chop_cost_volume_sample_coords_f32(void *stream, int half_centor, int64_t B, int64_t H,
                                       int64_t W, int64_t D, int64_t N, int64_t srcH,
                                       int64_t srcW, const float *base_plane,
                                       const float *offsets, const float *depth_grid,
                                       const float *Rs, const float *Ts, float *sw, float *sh,
                                       int32_t *fh, int32_t *fw, int32_t *state);
int chop_cost_volume_sample_coords_f64(void *stream, int half_centor, int64_t B, int64_t H,
                                       int64_t W, int64_t D, int64_t N, int64_t srcH,
                                       int64_t srcW, const double *base_plane,
                                       const double *offsets, const double *depth_grid,
                                       const double *Rs, const double *Ts, double *sw,
                                       double *sh, int32_t *fh, int32_t *fw, int32_t *state);

/* Selects the kernel family for subsequent calls from this thread: 0 = automatic (tiled
 * kernels where the shape allows, otherwise the strip kernels, otherwise the general
 * kernels), 1 = general kernels only, 2 = strip kernels where the shape allows (any storage
 * type, up to 64 channels), otherwise the general kernels.  Returns the previous value.  Used
 * by the tests to cover all three. */
int chop_set_kernel_family(int family);
/* Which family served the last forward/backward call of this thread: 0 none yet,
 * 1 general kernels, 2 tiled kernels, 3 strip kernels. */
int chop_last_kernel_family(void);
/* How many source views one workgroup of the last tiled backward call of this thread went
 * through in turn (1: every view had workgroups of its own; N: narrow pixels on a large
 * image, all views of a pixel tile in one workgroup); 0 if the last backward call did not run
 * the tiled kernels.  For the tests. */
int chop_last_views_per_workgroup(void);
/* No counterpart in the reference.  The tiled gradient kernels for 32 channels exist twice:
 * slimmed to four wavefronts per SIMD with a scatter window of 6 x 8 texels, and at three
 * wavefronts with 8 x 8.  The first is 8-11 % faster while the samples of consecutive depth
 * hypotheses land close to each other (ordinary rigs), the second about 9 % where they do not
 * (wide baselines with hypotheses close to the cameras).  The library cannot see the cameras
 * from the host and picks the second for five or more source views; rows = 6 or 8 fixes the
 * choice for subsequent calls from this thread, 0 returns it to the library.  Returns the
 * previous value.  Results agree within the gradient tolerance either way. */
int chop_set_backward_window(int rows);
/* Which of the two the last tiled backward call of this thread ran: 6 or 8; 0 for a shape
 * that has one kernel only, or if the last backward call did not run the tiled kernels.  For
 * the tests. */
int chop_last_backward_window(void);

#ifdef __cplusplus
}
#endif
#endif /* CHOP_COSTVOL_H_ */
