// Host-side plumbing shared by the C ABI (api.hip) and the kernel families
// (general.hip, tiled.hip): the argument block and the launcher prototypes.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "warp.h"

namespace chop {

// What the per-view term is and what a cost row holds:
//   SQUARED_DIFFERENCE      (sample - ref)^2 per channel              row = C values
//   GROUP_CORRELATION       sum over a channel group of sample * ref  row = groups values
//   SUM_SQUARED_DIFFERENCE  (sample - ref)^2 summed over the channels row = 1 value (CostAggregate)
//   BEST_GROUP_PAIR         largest correlation of any source group with any reference group
//                                                                     row = 1 value (CostVolumeV3)
//   WARP_ONLY               the sample itself, per view               row = N*C values (FeatureAggregate)
enum Corr {
  SQUARED_DIFFERENCE = 0,
  GROUP_CORRELATION = 1,
  SUM_SQUARED_DIFFERENCE = 2,
  BEST_GROUP_PAIR = 3,
  WARP_ONLY = 4
};

// Dynamic LDS a workgroup may ask for at launch without any per-kernel attribute having been
// set (HIP's limit on this hardware; the CU has 160 KiB).  Every kernel of the library stays
// inside it, so the launchers keep no state and may run on any number of host threads.
constexpr size_t kMaxDynamicLds = 64 * 1024;

// Channels per group the CostVolumeV3 kernels hold in registers (MAX_SUBCHANNELS_SIZE,
// custom_helper_op/cc/kernels/cost_volume_v3.h:35).
constexpr int kMaxSubChannels = 8;

// One call's arguments after validation.  S = storage type of the feature tensors,
// R = Storage<S>::Real = type of depth inputs, camera matrices, depth gradients.
template <typename S>
struct Args {
  using R = typename Storage<S>::Real;
  int64_t B, H, W, C, D, N, srcH, srcW;
  int groups;        // 1 for the squared-difference op
  int reduce;        // CHOP_REDUCE_MEAN / CHOP_REDUCE_MIN
  int corr;          // Corr
  R half;            // 0.5 or 0
  const S *ref, *src;
  const R *base_plane, *offsets;  // depth = base_plane[pixel] + offsets[b,d] ...
  const R *depth_grid;            // ... unless depth_grid != nullptr: depth_grid[voxel]
  const R *Rs, *Ts;
  // forward
  S *cost;
  int32_t *mask;
  // forward, optional (device scalar): stored instead of the cost wherever no view was
  // accepted (MEAN: count 0, MIN: winner -1) -- the cost-map layers' default fill
  // (custom_helper_op/python/layers/custom_layers.py:52-57, :78-83) folded into the store
  const R *default_cost;
  // backward
  const S *cost_grad;
  const int32_t *mask_in;
  S *ref_grad, *src_grad;
  R *depth_grad;  // [B,H,W] (base_plane) or [B,H,W,D] (depth_grid)
  // fp32 accumulation images for 16-bit storage (nullptr otherwise)
  float *ref_grad_acc, *src_grad_acc;

  __host__ __device__ int64_t pixels() const { return B * H * W; }
  __host__ __device__ int64_t voxels() const { return B * H * W * D; }
  __host__ __device__ int out_channels() const {
    return corr == GROUP_CORRELATION ? groups
           : corr == SUM_SQUARED_DIFFERENCE || corr == BEST_GROUP_PAIR ? 1
           : corr == WARP_ONLY ? (int)(N * C)
                               : (int)C;
  }
};

// One voxel of the sweep volume: indices, depth hypothesis and reference-pixel coordinates.
template <typename R>
struct Voxel {
  int64_t i, pix;
  int b, h, w, d;
  R depth, ref_w, ref_h;
};

template <typename S>
__device__ __forceinline__ Voxel<typename Storage<S>::Real> locate(const Args<S> &a, int64_t i) {
  using R = typename Storage<S>::Real;
  Voxel<R> v;
  v.i = i;
  v.pix = i / a.D;
  v.d = (int)(i - v.pix * a.D);
  const int64_t row = v.pix / a.W;
  v.w = (int)(v.pix - row * a.W);
  v.b = (int)(row / a.H);
  v.h = (int)(row - (int64_t)v.b * a.H);
  v.depth = a.depth_grid ? a.depth_grid[i] : a.base_plane[v.pix] + a.offsets[(int64_t)v.b * a.D + v.d];
  v.ref_w = static_cast<R>(v.w) + a.half;
  v.ref_h = static_cast<R>(v.h) + a.half;
  return v;
}

// General kernels: any shape, any channel count, both reduces, all storage types.
template <typename S>
hipError_t launch_general_forward(const Args<S> &a, hipStream_t stream);
template <typename S>
hipError_t launch_general_backward(const Args<S> &a, hipStream_t stream);

// Strip kernels: one wavefront per strip of pixels, one lane per channel, depth innermost.
// CostVolume, CostVolumeV2, CostAggregate and FeatureAggregate with up to 64 channels, any view
// count, all storage types: what the tiled kernels decline (float64, channel counts other than 4 x 2^k)
// runs here.
template <typename S>
bool strip_supported(const Args<S> &a);
// ... and the gradient of CostVolumeV3 (float, double; the forward pass has no strip kernel)
template <typename S>
bool strip_pair_backward_supported(const Args<S> &a);
template <typename S>
hipError_t launch_strip_forward(const Args<S> &a, hipStream_t stream);
template <typename S>
hipError_t launch_strip_backward(const Args<S> &a, hipStream_t stream);

// CostVolumeV3 (corr = BEST_GROUP_PAIR) and FeatureAggregate (corr = WARP_ONLY; `ref` unused,
// `cost` = mapped_feature [B,H,W,D,N,C], `mask` = mapped_mask [B,H,W,D,N]): float and double.
template <typename S>
hipError_t launch_v3_forward(const Args<S> &a, hipStream_t stream);
template <typename S>
hipError_t launch_v3_backward(const Args<S> &a, hipStream_t stream);
template <typename S>
hipError_t launch_feature_forward(const Args<S> &a, hipStream_t stream);
template <typename S>
hipError_t launch_feature_backward(const Args<S> &a, hipStream_t stream);

// Tiled kernels: wavefront-per-pixel-tile, depth innermost.  `supported` says whether the
// shape qualifies; the launchers must only be called when it does.
template <typename S>
bool tiled_forward_supported(const Args<S> &a);
template <typename S>
hipError_t launch_tiled_forward(const Args<S> &a, hipStream_t stream);
template <typename S>
bool tiled_backward_supported(const Args<S> &a);
template <typename S>
hipError_t launch_tiled_backward(const Args<S> &a, hipStream_t stream);
// Between the translation units of one direction and storage type: the kernels for 8 and 16
// lanes per pixel, where those are compiled apart from the rest.
template <typename S>
hipError_t launch_tiled_forward_wide(const Args<S> &a, hipStream_t stream);
template <typename S>
hipError_t launch_tiled_backward_wide(const Args<S> &a, hipStream_t stream);

// The tiled backward launcher reports how many views a workgroup took in turn (api.hip keeps
// it per host thread for chop_last_views_per_workgroup).
void note_views_per_workgroup(int views);
// The calling thread's choice between the two 32-channel tiled gradient kernels
// (chop_set_backward_window): 0 the launcher decides, 6 slimmed, 8 wide.
int backward_window_mode();
// ... and which of the two the launcher took (0: a shape that has only one kernel)
void note_backward_window(int rows);

// Utility launches.
hipError_t launch_fill_zero(void *ptr, size_t bytes, hipStream_t stream);
// Up to three ranges zeroed by ONE launch (a launch costs ~5 us, the ranges are small):
// collect them with add(), then launch().
struct ZeroRanges {
  static constexpr int kMax = 3;
  unsigned char *ptr[kMax] = {nullptr, nullptr, nullptr};
  size_t bytes[kMax] = {0, 0, 0};
  int count = 0;
  bool bad = false;  // a range too many, or a NULL pointer with bytes: launch() reports it
  void add(void *p, size_t n) {
    if (n == 0) return;
    if (count >= kMax || p == nullptr) {
      bad = true;
      return;
    }
    ptr[count] = static_cast<unsigned char *>(p);
    bytes[count] = n;
    ++count;
  }
  hipError_t launch(hipStream_t stream) const;  // hipErrorInvalidValue when `bad`
};
template <typename S>
hipError_t launch_narrow(const float *from, S *to, int64_t count, hipStream_t stream);
// two fp32 images narrowed to 16-bit storage by one launch
template <typename S>
hipError_t launch_narrow2(const float *from0, S *to0, int64_t count0, const float *from1, S *to1,
                          int64_t count1, hipStream_t stream);

template <typename R>
hipError_t launch_sample_coords(R half, int64_t B, int64_t H, int64_t W, int64_t D, int64_t N,
                                int64_t srcH, int64_t srcW, const R *base_plane,
                                const R *offsets, const R *depth_grid, const R *Rs, const R *Ts,
                                R *sw, R *sh, int32_t *fh, int32_t *fw, int32_t *state,
                                hipStream_t stream);

// CostMapLayer's default fill and its gradient; the relative projection of a camera pair.
template <typename R>
hipError_t launch_default_fill(int reduce, int64_t mask_count, int64_t inner, const R *cost,
                               const int32_t *mask, const R *default_cost, R *out,
                               hipStream_t stream);
// (S: float, double, or a 16-bit storage type whose sum is kept in float)
template <typename S>
hipError_t launch_default_fill_grad(int reduce, int64_t mask_count, int64_t inner,
                                    const S *out_grad, const int32_t *mask, S *cost_grad,
                                    typename Storage<S>::Real *default_grad, hipStream_t stream);
template <typename R>
hipError_t launch_combine_projection(int64_t B, int64_t N, const R *ref_cam, const R *src_cam,
                                     const R *scale, R *Rs, R *Ts, hipStream_t stream);

int grid_for(int64_t work_items, int block);

}  // namespace chop
