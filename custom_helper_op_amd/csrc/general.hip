// General cost-volume kernels: one thread per (voxel, output channel).  They accept any
// channel count, view count and storage type and both reduce methods; the tiled kernels
// take over for the shapes they are specialised for.  The arithmetic is the reference's
// literal operand order with every operation rounded separately, so for float and double
// the forward results are bit-identical to a plain IEEE CPU evaluation of
// custom_helper_op/cc/kernels/cost_volume_kernels_gpu.cu.cc:33-228 and
// cost_volume_kernels_gpu_v2.cu.cc:33-235.
#include <algorithm>
#include <type_traits>

#include "internal.h"

namespace chop {

namespace {

constexpr int kBlock = 256;

template <typename S>
struct Is16 : std::integral_constant<bool, sizeof(S) == 2> {};

template <typename S, int CORR, int REDUCE>
__global__ __launch_bounds__(kBlock) void general_forward_kernel(const Args<S> a) {
  using R = typename Storage<S>::Real;
  const int C = (int)a.C, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW;
  const int OC = CORR ? a.groups : C;
  const int sub = CORR ? C / a.groups : 1;
  const int64_t total = a.voxels() * OC;
  const int64_t row_step = (int64_t)srcW * C;
  for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * kBlock) {
    const int64_t i = e / OC;
    const int oc = (int)(e - i * OC);
    const Voxel<R> v = locate(a, i);
    const S *ref_px = a.ref + v.pix * C;
    R acc = REDUCE == 0 ? R(0) : (CORR ? Limits<R>::min_positive() : Limits<R>::max());
    int arg = -1, used = 0;
    for (int n = 0; n < N; ++n) {
      Sample<R> s;
      const int64_t cam = (int64_t)v.b * N + n;
      project(a.Rs + cam * 9, a.Ts + cam * 3, v.ref_w, v.ref_h, v.depth, a.half, srcH, srcW, s);
      if (s.state != 2) continue;
      const S *t00 = a.src + (int64_t)C * (s.fw + (int64_t)srcW * (s.fh + (int64_t)srcH * cam));
      const S *t01 = t00 + C, *t11 = t01 + row_step, *t10 = t00 + row_step;
      R val;
      if (CORR == 0) {
        const R smp = s.k00 * Storage<S>::load(t00 + oc) + s.k01 * Storage<S>::load(t01 + oc) +
                      s.k11 * Storage<S>::load(t11 + oc) + s.k10 * Storage<S>::load(t10 + oc);
        const R diff = smp - Storage<S>::load(ref_px + oc);
        val = diff * diff;
      } else {
        val = R(0);
        for (int c = oc * sub; c < oc * sub + sub; ++c) {
          const R smp = s.k00 * Storage<S>::load(t00 + c) + s.k01 * Storage<S>::load(t01 + c) +
                        s.k11 * Storage<S>::load(t11 + c) + s.k10 * Storage<S>::load(t10 + c);
          val += smp * Storage<S>::load(ref_px + c);
        }
      }
      if (REDUCE == 0) {
        acc += val;
      } else if (CORR ? (acc < val) : (acc > val)) {
        acc = val;
        arg = n;
      }
      ++used;
    }
    if (REDUCE == 0) {
      if (used > 0) acc = acc / static_cast<R>(used);
      if (oc == 0) a.mask[i] = used;
    } else {
      a.mask[e] = arg;
    }
    if (a.default_cost != nullptr && (REDUCE == 0 ? used == 0 : arg < 0)) acc = *a.default_cost;
    Storage<S>::store(a.cost + e, acc);
  }
}

// CostAggregate forward: one thread per voxel, channels and views serial, in the order of
// cost_aggregate_kernels_gpu.cu.cc:75-124 (MEAN) and :173-228 (MIN).
template <typename S, int REDUCE>
__global__ __launch_bounds__(kBlock) void general_aggregate_forward_kernel(const Args<S> a) {
  using R = typename Storage<S>::Real;
  const int C = (int)a.C, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW;
  const int64_t total = a.voxels();
  const int64_t row_step = (int64_t)srcW * C;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * kBlock) {
    const Voxel<R> v = locate(a, i);
    const S *ref_px = a.ref + v.pix * C;
    R acc = REDUCE == 0 ? R(0) : Limits<R>::max();
    int used = REDUCE == 0 ? 0 : -1;
    for (int n = 0; n < N; ++n) {
      Sample<R> s;
      const int64_t cam = (int64_t)v.b * N + n;
      project(a.Rs + cam * 9, a.Ts + cam * 3, v.ref_w, v.ref_h, v.depth, a.half, srcH, srcW, s);
      if (s.state != 2) continue;
      const S *t00 = a.src + (int64_t)C * (s.fw + (int64_t)srcW * (s.fh + (int64_t)srcH * cam));
      const S *t01 = t00 + C, *t11 = t01 + row_step, *t10 = t00 + row_step;
      R cur = REDUCE == 0 ? acc : R(0);
      for (int c = 0; c < C; ++c) {
        const R smp = s.k00 * Storage<S>::load(t00 + c) + s.k01 * Storage<S>::load(t01 + c) +
                      s.k11 * Storage<S>::load(t11 + c) + s.k10 * Storage<S>::load(t10 + c);
        const R diff = smp - Storage<S>::load(ref_px + c);
        cur += diff * diff;
      }
      if (REDUCE == 0) {
        acc = cur;
        ++used;
      } else if (acc > cur) {
        acc = cur;
        used = n;
      }
    }
    a.mask[i] = used;
    R out = R(0);
    if (REDUCE == 0) {
      if (used > 0) out = acc / static_cast<R>((int64_t)used * C);
    } else if (used >= 0) {
      out = acc / static_cast<R>(C);
    }
    if (a.default_cost != nullptr && (REDUCE == 0 ? used <= 0 : used < 0)) out = *a.default_cost;
    Storage<S>::store(a.cost + i, out);
  }
}

template <typename S, int CORR, int REDUCE>
__global__ __launch_bounds__(kBlock) void general_backward_kernel(const Args<S> a) {
  using R = typename Storage<S>::Real;
  using Acc = typename std::conditional<Is16<S>::value, float, S>::type;
  Acc *ref_grad = Is16<S>::value ? (Acc *)a.ref_grad_acc : (Acc *)a.ref_grad;
  Acc *src_grad = Is16<S>::value ? (Acc *)a.src_grad_acc : (Acc *)a.src_grad;
  const int C = (int)a.C, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW;
  // CORR == 2 (CostAggregate, cost_aggregate_kernels_gpu.cu.cc:338-563): one upstream
  // gradient and one mask entry per voxel, shared by all channels
  const int OC = CORR == 1 ? a.groups : CORR == 2 ? 1 : C;
  const int sub = CORR == 1 ? C / a.groups : 1;
  const int64_t total = a.voxels() * C;
  const int64_t row_step = (int64_t)srcW * C;
  for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * kBlock) {
    const int64_t i = e / C;
    const int c = (int)(e - i * C);
    const int oc = CORR == 1 ? c / sub : CORR == 2 ? 0 : c;
    const int32_t *mrow = a.mask_in + (REDUCE == 0 ? i : i * OC);
    const int32_t m0 = mrow[0];
    if (REDUCE == 0 ? (m0 <= 0) : (m0 < 0)) continue;  // depth gradient stays at its zero fill
    const int32_t winner = REDUCE == 0 ? 0 : mrow[oc];
    const Voxel<R> v = locate(a, i);
    const R ref_c = Storage<S>::load(a.ref + v.pix * C + c);
    R cg = Storage<S>::load(a.cost_grad + i * OC + oc);
    if (CORR == 2)  // :388 cost_grad / (T)(mask * channels), :502 cost_grad / (T)channels
      cg = REDUCE == 0 ? cg / static_cast<R>((int64_t)m0 * C) : cg / static_cast<R>(C);
    R depth_grad = R(0);
    for (int n = 0; n < N; ++n) {
      Sample<R> s;
      const int64_t cam = (int64_t)v.b * N + n;
      project(a.Rs + cam * 9, a.Ts + cam * 3, v.ref_w, v.ref_h, v.depth, a.half, srcH, srcW, s);
      if (s.state != 2) continue;
      if (REDUCE != 0 && winner != n) continue;
      const int64_t off = (int64_t)C * (s.fw + (int64_t)srcW * (s.fh + (int64_t)srcH * cam)) + c;
      const R v00 = Storage<S>::load(a.src + off), v01 = Storage<S>::load(a.src + off + C),
              v11 = Storage<S>::load(a.src + off + C + row_step),
              v10 = Storage<S>::load(a.src + off + row_step);
      const R smp = s.k00 * v00 + s.k01 * v01 + s.k11 * v11 + s.k10 * v10;
      R g;
      if (CORR == 0) {
        const R diff = smp - ref_c;
        g = REDUCE == 0 ? R(2) * diff * cg / static_cast<R>(m0) : R(2) * diff * cg;
        atomic_add(ref_grad + v.pix * C + c, (Acc)(-g));
      } else if (CORR == 2) {
        const R diff = smp - ref_c;
        g = R(2) * diff * cg;
        atomic_add(ref_grad + v.pix * C + c, (Acc)(-g));
      } else {
        g = REDUCE == 0 ? cg / static_cast<R>(m0) : cg;
        atomic_add(ref_grad + v.pix * C + c, (Acc)(g * smp));
        g = g * ref_c;
      }
      atomic_add(src_grad + off, (Acc)(g * s.k00));
      atomic_add(src_grad + off + C, (Acc)(g * s.k01));
      atomic_add(src_grad + off + C + row_step, (Acc)(g * s.k11));
      atomic_add(src_grad + off + row_step, (Acc)(g * s.k10));
      const R t1 = v11 - v10 - v01 + v00;
      const R h_grad = g * (t1 * s.dw + v10 - v00);
      const R w_grad = g * (t1 * s.dh + v01 - v00);
      depth_grad += depth_chain(s, h_grad, w_grad);
    }
    if (a.depth_grad) atomic_add(a.depth_grad + (a.depth_grid ? i : v.pix), depth_grad);
  }
}

__device__ __forceinline__ void zero_range(unsigned char *p, size_t bytes) {
  // head up to 16-byte alignment, 16-byte body, byte tail
  const size_t mis = (size_t)(-(intptr_t)p) & 15u;
  const size_t head = mis < bytes ? mis : bytes;
  const size_t body = (bytes - head) / 16;
  const size_t tid = (size_t)blockIdx.x * kBlock + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * kBlock;
  uint4 *q = reinterpret_cast<uint4 *>(p + head);
  const uint4 z = make_uint4(0, 0, 0, 0);
  for (size_t k = tid; k < body; k += stride) q[k] = z;
  const size_t tail_at = head + body * 16;
  if (tid < head) p[tid] = 0;
  if (tid < bytes - tail_at) p[tail_at + tid] = 0;
}

__global__ __launch_bounds__(kBlock) void fill_zero_kernel(unsigned char *p, size_t bytes) {
  zero_range(p, bytes);
}

__global__ __launch_bounds__(kBlock) void fill_zero_ranges_kernel(const ZeroRanges r) {
  for (int i = 0; i < r.count; ++i) zero_range(r.ptr[i], r.bytes[i]);
}

// fp32 accumulation images to their 16-bit outputs.  A thread takes eight consecutive elements:
// two 16-byte loads that bypass the caches (an accumulator is read exactly once) and one
// 16-byte store; with one element per thread the 2-byte stores held the pass to half the
// stream rate.  `vec` = both pointers 16-byte aligned (else element by element).
template <typename S>
__device__ __forceinline__ void narrow_range(const float *from, S *to, int64_t count, bool vec,
                                             int64_t tid, int64_t stride) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  const int64_t octets = vec ? count / 8 : 0;
  for (int64_t k = tid; k < octets; k += stride) {
    const f32x4 lo = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(from) + 2 * k);
    const f32x4 hi = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(from) + 2 * k + 1);
    S out[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) Storage<S>::store(out + i, lo[i]), Storage<S>::store(out + 4 + i, hi[i]);
    *(reinterpret_cast<u32x4 *>(to) + k) = *reinterpret_cast<const u32x4 *>(out);
  }
  for (int64_t k = octets * 8 + tid; k < count; k += stride) Storage<S>::store(to + k, from[k]);
}

template <typename S>
__global__ __launch_bounds__(kBlock) void narrow_kernel(const float *from, S *to, int64_t count,
                                                        bool vec) {
  narrow_range<S>(from, to, count, vec, (int64_t)blockIdx.x * kBlock + threadIdx.x,
                  (int64_t)gridDim.x * kBlock);
}

template <typename S>
__global__ __launch_bounds__(kBlock) void narrow2_kernel(const float *from0, S *to0, int64_t count0,
                                                         bool vec0, const float *from1, S *to1,
                                                         int64_t count1, bool vec1) {
  const int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x, stride = (int64_t)gridDim.x * kBlock;
  narrow_range<S>(from0, to0, count0, vec0, tid, stride);
  narrow_range<S>(from1, to1, count1, vec1, tid, stride);
}

template <typename R>
__global__ __launch_bounds__(kBlock) void sample_coords_kernel(
    R half, int64_t H, int64_t W, int64_t D, int64_t N, int srcH, int srcW, int64_t total,
    const R *base_plane, const R *offsets, const R *depth_grid, const R *Rs, const R *Ts, R *sw,
    R *sh, int32_t *fh, int32_t *fw, int32_t *state) {
  for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * kBlock) {
    const int64_t i = e / N;
    const int n = (int)(e - i * N);
    const int64_t pix = i / D;
    const int d = (int)(i - pix * D);
    const int64_t row = pix / W;
    const int w = (int)(pix - row * W);
    const int64_t b = row / H;
    const int h = (int)(row - b * H);
    const R depth = depth_grid ? depth_grid[i] : base_plane[pix] + offsets[b * D + d];
    Sample<R> s;
    const int64_t cam = b * N + n;
    project(Rs + cam * 9, Ts + cam * 3, static_cast<R>(w) + half, static_cast<R>(h) + half, depth,
            half, srcH, srcW, s);
    sw[e] = s.sw;
    sh[e] = s.sh;
    fh[e] = s.fh;
    fw[e] = s.fw;
    state[e] = s.state;
  }
}

}  // namespace

int grid_for(int64_t work_items, int block) {
  const int64_t blocks = (work_items + block - 1) / block;
  return (int)std::max<int64_t>(1, std::min<int64_t>(blocks, 1 << 16));
}

hipError_t launch_fill_zero(void *ptr, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  fill_zero_kernel<<<grid_for((int64_t)(bytes / 16 + 32), kBlock), kBlock, 0, stream>>>(
      static_cast<unsigned char *>(ptr), bytes);
  return hipGetLastError();
}

hipError_t ZeroRanges::launch(hipStream_t stream) const {
  if (bad) return hipErrorInvalidValue;
  if (count == 0) return hipSuccess;
  size_t most = 0;
  for (int i = 0; i < count; ++i) most = bytes[i] > most ? bytes[i] : most;
  fill_zero_ranges_kernel<<<grid_for((int64_t)(most / 16 + 32), kBlock), kBlock, 0, stream>>>(*this);
  return hipGetLastError();
}

inline bool both_aligned16(const void *a, const void *b) {
  return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
}

template <typename S>
hipError_t launch_narrow2(const float *from0, S *to0, int64_t count0, const float *from1, S *to1,
                          int64_t count1, hipStream_t stream) {
  const int64_t most = count0 > count1 ? count0 : count1;
  if (most == 0) return hipSuccess;
  narrow2_kernel<S><<<grid_for((most + 7) / 8, kBlock), kBlock, 0, stream>>>(
      from0, to0, count0, both_aligned16(from0, to0), from1, to1, count1, both_aligned16(from1, to1));
  return hipGetLastError();
}
template hipError_t launch_narrow2<__half>(const float *, __half *, int64_t, const float *, __half *,
                                           int64_t, hipStream_t);
template hipError_t launch_narrow2<bf16_t>(const float *, bf16_t *, int64_t, const float *, bf16_t *,
                                           int64_t, hipStream_t);

template <typename S>
hipError_t launch_narrow(const float *from, S *to, int64_t count, hipStream_t stream) {
  if (count == 0) return hipSuccess;
  narrow_kernel<S><<<grid_for((count + 7) / 8, kBlock), kBlock, 0, stream>>>(from, to, count,
                                                                             both_aligned16(from, to));
  return hipGetLastError();
}
template hipError_t launch_narrow<__half>(const float *, __half *, int64_t, hipStream_t);
template hipError_t launch_narrow<bf16_t>(const float *, bf16_t *, int64_t, hipStream_t);

template <typename S>
hipError_t launch_general_forward(const Args<S> &a, hipStream_t stream) {
  const int64_t total = a.voxels() * a.out_channels();
  if (total == 0) return hipSuccess;
  const int grid = grid_for(total, kBlock);
  if (a.corr == SUM_SQUARED_DIFFERENCE) {
    if (a.reduce == 0)
      general_aggregate_forward_kernel<S, 0><<<grid, kBlock, 0, stream>>>(a);
    else
      general_aggregate_forward_kernel<S, 1><<<grid, kBlock, 0, stream>>>(a);
  } else if (a.corr == SQUARED_DIFFERENCE) {
    if (a.reduce == 0)
      general_forward_kernel<S, 0, 0><<<grid, kBlock, 0, stream>>>(a);
    else
      general_forward_kernel<S, 0, 1><<<grid, kBlock, 0, stream>>>(a);
  } else {
    if (a.reduce == 0)
      general_forward_kernel<S, 1, 0><<<grid, kBlock, 0, stream>>>(a);
    else
      general_forward_kernel<S, 1, 1><<<grid, kBlock, 0, stream>>>(a);
  }
  return hipGetLastError();
}

template <typename S>
hipError_t launch_general_backward(const Args<S> &a, hipStream_t stream) {
  using R = typename Storage<S>::Real;
  const int64_t n_ref = a.pixels() * a.C;
  const int64_t n_src = a.B * a.N * a.srcH * a.srcW * a.C;
  const int64_t n_depth = a.depth_grid ? a.voxels() : a.pixels();
  hipError_t err;
  ZeroRanges zero;  // everything the kernel accumulates into, one launch
  if (Is16<S>::value) {
    zero.add(a.ref_grad_acc, (size_t)n_ref * 4);
    zero.add(a.src_grad_acc, (size_t)n_src * 4);
  } else {
    zero.add(a.ref_grad, (size_t)n_ref * sizeof(S));
    zero.add(a.src_grad, (size_t)n_src * sizeof(S));
  }
  if (a.depth_grad != nullptr) zero.add(a.depth_grad, (size_t)n_depth * sizeof(R));
  if ((err = zero.launch(stream)) != hipSuccess) return err;
  const int64_t total = a.voxels() * a.C;
  if (total > 0) {
    const int grid = grid_for(total, kBlock);
    if (a.corr == SUM_SQUARED_DIFFERENCE) {
      if (a.reduce == 0)
        general_backward_kernel<S, 2, 0><<<grid, kBlock, 0, stream>>>(a);
      else
        general_backward_kernel<S, 2, 1><<<grid, kBlock, 0, stream>>>(a);
    } else if (a.corr == SQUARED_DIFFERENCE) {
      if (a.reduce == 0)
        general_backward_kernel<S, 0, 0><<<grid, kBlock, 0, stream>>>(a);
      else
        general_backward_kernel<S, 0, 1><<<grid, kBlock, 0, stream>>>(a);
    } else {
      if (a.reduce == 0)
        general_backward_kernel<S, 1, 0><<<grid, kBlock, 0, stream>>>(a);
      else
        general_backward_kernel<S, 1, 1><<<grid, kBlock, 0, stream>>>(a);
    }
    if ((err = hipGetLastError()) != hipSuccess) return err;
  }
  if constexpr (Is16<S>::value) {
    if ((err = launch_narrow2<S>(a.ref_grad_acc, a.ref_grad, n_ref, a.src_grad_acc, a.src_grad, n_src,
                                 stream)) != hipSuccess)
      return err;
  }
  return hipSuccess;
}

template <typename R>
hipError_t launch_sample_coords(R half, int64_t B, int64_t H, int64_t W, int64_t D, int64_t N,
                                int64_t srcH, int64_t srcW, const R *base_plane,
                                const R *offsets, const R *depth_grid, const R *Rs, const R *Ts,
                                R *sw, R *sh, int32_t *fh, int32_t *fw, int32_t *state,
                                hipStream_t stream) {
  const int64_t total = B * H * W * D * N;
  if (total == 0) return hipSuccess;
  sample_coords_kernel<R><<<grid_for(total, kBlock), kBlock, 0, stream>>>(
      half, H, W, D, N, (int)srcH, (int)srcW, total, base_plane, offsets, depth_grid, Rs, Ts, sw,
      sh, fh, fw, state);
  return hipGetLastError();
}

#define CHOP_INSTANTIATE(S)                                                        \
  template hipError_t launch_general_forward<S>(const Args<S> &, hipStream_t);     \
  template hipError_t launch_general_backward<S>(const Args<S> &, hipStream_t);
CHOP_INSTANTIATE(float)
CHOP_INSTANTIATE(double)
CHOP_INSTANTIATE(__half)
CHOP_INSTANTIATE(bf16_t)
#undef CHOP_INSTANTIATE

template hipError_t launch_sample_coords<float>(float, int64_t, int64_t, int64_t, int64_t, int64_t,
                                                int64_t, int64_t, const float *, const float *,
                                                const float *, const float *, const float *,
                                                float *, float *, int32_t *, int32_t *, int32_t *,
                                                hipStream_t);
template hipError_t launch_sample_coords<double>(double, int64_t, int64_t, int64_t, int64_t,
                                                 int64_t, int64_t, int64_t, const double *,
                                                 const double *, const double *, const double *,
                                                 const double *, double *, double *, int32_t *,
                                                 int32_t *, int32_t *, hipStream_t);

}  // namespace chop
