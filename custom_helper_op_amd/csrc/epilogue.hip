// The callers on either side of the cost-volume ops, as small kernels:
//
//  * default fill: CostMapLayer / CostMapLayerV2 replace the cost of a voxel that no view
//    covered by a (trainable) scalar, `tf.where(cost_mask > 0, cost, default)` for the mean
//    and `cost_mask >= 0` for the minimum (custom_helper_op/python/layers/
//    custom_layers.py:52-57, :78-83).  The gradient of `where` sends the upstream gradient to
//    the cost where the mask holds and sums it into the scalar's gradient where it does not.
//  * combine_projection: the relative projection (Rs, Ts) the ops take, from the reference
//    and source cameras' extrinsics and intrinsics
//    (custom_helper_op/python/ops/op_tests/cost_volume_op_test.py:115-134).
#include <algorithm>

#include "internal.h"

namespace chop {

namespace {

constexpr int kBlock = 256;

template <typename R>
__global__ __launch_bounds__(kBlock) void default_fill_kernel(int reduce, int64_t total,
                                                              int64_t inner, const R *cost,
                                                              const int32_t *mask,
                                                              const R *default_cost, R *out) {
  const R fill = *default_cost;
  for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * kBlock) {
    const int32_t m = mask[e / inner];
    const bool keep = reduce == 0 ? m > 0 : m >= 0;
    out[e] = keep ? cost[e] : fill;
  }
}

template <typename S, typename R>
__global__ __launch_bounds__(kBlock) void default_fill_grad_kernel(int reduce, int64_t total,
                                                                   int64_t inner,
                                                                   const S *out_grad,
                                                                   const int32_t *mask,
                                                                   S *cost_grad, R *default_grad) {
  __shared__ R partial[kBlock / 64];
  R sum = R(0);
  for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * kBlock) {
    const int32_t m = mask[e / inner];
    const bool keep = reduce == 0 ? m > 0 : m >= 0;
    const R g = Storage<S>::load(out_grad + e);  // (16-bit storage: summed in float)
    if (cost_grad != nullptr) Storage<S>::store(cost_grad + e, keep ? g : R(0));
    if (!keep) sum += g;
  }
  // wavefront sum, then one atomic per workgroup
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_down(sum, off, 64);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    R tot = R(0);
#pragma unroll
    for (int k = 0; k < kBlock / 64; ++k) tot += partial[k];
    if (tot != R(0)) atomic_add(default_grad, tot);
  }
}

template <typename R>
__device__ __forceinline__ void mat3_mul(const R *a, const R *b, R *out) {
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j)
      out[i * 3 + j] = a[i * 3] * b[j] + a[i * 3 + 1] * b[3 + j] + a[i * 3 + 2] * b[6 + j];
}

// One thread per (batch item, source view).  cam = [2,4,4]: extrinsic [R|t] then intrinsic K
// in the upper-left 3x3 (the layout of the reference's load_cam, cost_volume_op_test.py:75-113).
template <typename R>
__global__ __launch_bounds__(64) void combine_projection_kernel(int64_t total, int64_t N,
                                                                const R *ref_cam,
                                                                const R *src_cam, const R *scale,
                                                                R *Rs, R *Ts) {
  const int64_t e = (int64_t)blockIdx.x * 64 + threadIdx.x;
  if (e >= total) return;
  const R *rc = ref_cam + (e / N) * 32, *sc = src_cam + e * 32;
  R refR[9], refT[3], refK[9], srcR[9], srcT[3], srcK[9];
#pragma unroll
  for (int i = 0; i < 3; ++i) {
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      refR[i * 3 + j] = rc[i * 4 + j];
      srcR[i * 3 + j] = sc[i * 4 + j];
      refK[i * 3 + j] = rc[16 + i * 4 + j] * scale[i];  // K * scale[:, None]
      srcK[i * 3 + j] = sc[16 + i * 4 + j] * scale[i];
    }
    refT[i] = rc[i * 4 + 3];
    srcT[i] = sc[i * 4 + 3];
  }
  refK[2] += R(0.5), refK[5] += R(0.5), srcK[2] += R(0.5), srcK[5] += R(0.5);  // :125-128
  // inverse of ref_K by cofactors
  const R c00 = refK[4] * refK[8] - refK[5] * refK[7], c01 = refK[5] * refK[6] - refK[3] * refK[8],
          c02 = refK[3] * refK[7] - refK[4] * refK[6];
  const R det = refK[0] * c00 + refK[1] * c01 + refK[2] * c02;
  const R inv = R(1) / det;
  R Kinv[9];
  Kinv[0] = c00 * inv, Kinv[3] = c01 * inv, Kinv[6] = c02 * inv;
  Kinv[1] = (refK[2] * refK[7] - refK[1] * refK[8]) * inv;
  Kinv[4] = (refK[0] * refK[8] - refK[2] * refK[6]) * inv;
  Kinv[7] = (refK[1] * refK[6] - refK[0] * refK[7]) * inv;
  Kinv[2] = (refK[1] * refK[5] - refK[2] * refK[4]) * inv;
  Kinv[5] = (refK[2] * refK[3] - refK[0] * refK[5]) * inv;
  Kinv[8] = (refK[0] * refK[4] - refK[1] * refK[3]) * inv;
  R refRt[9], dR[9], tmp[9], out[9];
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j) refRt[i * 3 + j] = refR[j * 3 + i];
  mat3_mul(srcR, refRt, dR);   // delta_R = src_R ref_R^T          (:132)
  mat3_mul(dR, Kinv, tmp);     // delta_R ref_K^-1
  mat3_mul(srcK, tmp, out);    // R = src_K (delta_R ref_K^-1)      (:134)
  R dT[3];
#pragma unroll
  for (int i = 0; i < 3; ++i)  // delta_T = src_T - delta_R ref_T   (:133)
    dT[i] = srcT[i] - (dR[i * 3] * refT[0] + dR[i * 3 + 1] * refT[1] + dR[i * 3 + 2] * refT[2]);
#pragma unroll
  for (int k = 0; k < 9; ++k) Rs[e * 9 + k] = out[k];
#pragma unroll
  for (int i = 0; i < 3; ++i)  // T = src_K delta_T                 (:135)
    Ts[e * 3 + i] = srcK[i * 3] * dT[0] + srcK[i * 3 + 1] * dT[1] + srcK[i * 3 + 2] * dT[2];
}

}  // namespace

template <typename R>
hipError_t launch_default_fill(int reduce, int64_t mask_count, int64_t inner, const R *cost,
                               const int32_t *mask, const R *default_cost, R *out,
                               hipStream_t stream) {
  const int64_t total = mask_count * inner;
  if (total == 0) return hipSuccess;
  default_fill_kernel<R><<<grid_for(total, kBlock), kBlock, 0, stream>>>(reduce, total, inner, cost,
                                                                       mask, default_cost, out);
  return hipGetLastError();
}

template <typename S>
hipError_t launch_default_fill_grad(int reduce, int64_t mask_count, int64_t inner,
                                    const S *out_grad, const int32_t *mask, S *cost_grad,
                                    typename Storage<S>::Real *default_grad, hipStream_t stream) {
  using R = typename Storage<S>::Real;
  hipError_t err = launch_fill_zero(default_grad, sizeof(R), stream);
  if (err != hipSuccess) return err;
  const int64_t total = mask_count * inner;
  if (total == 0) return hipSuccess;
  const int grid = (int)std::min<int64_t>(grid_for(total, kBlock), 2048);
  default_fill_grad_kernel<S, R><<<grid, kBlock, 0, stream>>>(reduce, total, inner, out_grad, mask,
                                                             cost_grad, default_grad);
  return hipGetLastError();
}

template <typename R>
hipError_t launch_combine_projection(int64_t B, int64_t N, const R *ref_cam, const R *src_cam,
                                     const R *scale, R *Rs, R *Ts, hipStream_t stream) {
  const int64_t total = B * N;
  if (total == 0) return hipSuccess;
  combine_projection_kernel<R><<<(unsigned)((total + 63) / 64), 64, 0, stream>>>(
      total, N, ref_cam, src_cam, scale, Rs, Ts);
  return hipGetLastError();
}

#define CHOP_INSTANTIATE(R)                                                                      \
  template hipError_t launch_default_fill<R>(int, int64_t, int64_t, const R *, const int32_t *,  \
                                             const R *, R *, hipStream_t);                       \
  template hipError_t launch_default_fill_grad<R>(int, int64_t, int64_t, const R *,              \
                                                  const int32_t *, R *, R *, hipStream_t);       \
  template hipError_t launch_combine_projection<R>(int64_t, int64_t, const R *, const R *,       \
                                                   const R *, R *, R *, hipStream_t);
CHOP_INSTANTIATE(float)
CHOP_INSTANTIATE(double)
#undef CHOP_INSTANTIATE
template hipError_t launch_default_fill_grad<__half>(int, int64_t, int64_t, const __half *,
                                                     const int32_t *, __half *, float *, hipStream_t);
template hipError_t launch_default_fill_grad<bf16_t>(int, int64_t, int64_t, const bf16_t *,
                                                     const int32_t *, bf16_t *, float *, hipStream_t);

}  // namespace chop
