// CostVolumeV3 and FeatureAggregate: general kernels (any shape, float and double).
//
// CostVolumeV3 (custom_helper_op/cc/kernels/cost_volume_kernels_gpu_v3.cu.cc:33-261, 376-639):
// per accepted view the largest dot product between any channel group of the bilinear sample
// and any channel group of the reference pixel; MEAN averages the views' maxima, MIN keeps the
// overall maximum and records (view, reference group, source group).  One thread per voxel:
// the winner of a voxel is an index triple, so the pairs are visited in the reference's order
// with its strict comparison, every product and sum rounded separately.
//
// FeatureAggregate (feature_aggregate_kernels_gpu.cu.cc:33-121, 219-326): the warp alone,
// mapped_feature[B,H,W,D,N,C] and a 0/1 mask per (voxel, view).  One thread per (voxel, view,
// channel slice); a slice is 16 bytes when the channel count and the pointers allow.
#include <type_traits>

#include "internal.h"

namespace chop {

namespace {

constexpr int kBlock = 256;

template <typename R>
struct Taps {
  const R *t00, *t01, *t11, *t10;
};

template <typename R>
__device__ __forceinline__ Taps<R> taps_of(const R *src, const Sample<R> &s, int64_t cam, int C,
                                           int srcH, int srcW) {
  Taps<R> t;
  t.t00 = src + (int64_t)C * (s.fw + (int64_t)srcW * (s.fh + (int64_t)srcH * cam));
  t.t01 = t.t00 + C;
  t.t11 = t.t01 + (int64_t)srcW * C;
  t.t10 = t.t00 + (int64_t)srcW * C;
  return t;
}

// ---- 16-byte slices of a channel row ------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename R, int VEC>
struct Slice {
  R v[VEC];
};

template <typename R, int VEC>
__device__ __forceinline__ Slice<R, VEC> load_slice(const R *p) {
  Slice<R, VEC> out;
  if constexpr (VEC * sizeof(R) == 16) {
    const u32x4 raw = *reinterpret_cast<const u32x4 *>(p);
    __builtin_memcpy(out.v, &raw, 16);
  } else {
#pragma unroll
    for (int k = 0; k < VEC; ++k) out.v[k] = p[k];
  }
  return out;
}

template <typename R, int VEC>
__device__ __forceinline__ void store_slice(R *p, const Slice<R, VEC> &in) {
  if constexpr (VEC * sizeof(R) == 16) {
    u32x4 raw;
    __builtin_memcpy(&raw, in.v, 16);
    __builtin_nontemporal_store(raw, reinterpret_cast<u32x4 *>(p));  // written once, never re-read
  } else {
#pragma unroll
    for (int k = 0; k < VEC; ++k) p[k] = in.v[k];
  }
}

// Best (source group, reference group) pair of one accepted sample: source group outermost,
// strict "<", seeded with `seed` (cost_volume_kernels_gpu_v3.cu.cc:113-130, 231-250).
// gi, gs are left untouched when no pair exceeds the seed.
// SUB: channels per group when that is 4 or 8 floats and every row is 16-byte aligned (the
// taps and the reference groups are then fetched with 16-byte loads), 0 for any other case.
// The arithmetic is the same expression per element either way.
template <typename R, int SUB>
__device__ __forceinline__ R best_pair(const Sample<R> &s, const Taps<R> &t, const R *ref_px,
                                       int groups, int sub, R seed, int &gi_out, int &gs_out) {
  R buf[kMaxSubChannels];
  R best = seed;
  for (int gs = 0; gs < groups; ++gs) {
    if constexpr (SUB > 0) {
#pragma unroll
      for (int k0 = 0; k0 < SUB; k0 += 4) {
        const int sc = gs * SUB + k0;
        const Slice<R, 4> v00 = load_slice<R, 4>(t.t00 + sc), v01 = load_slice<R, 4>(t.t01 + sc),
                          v11 = load_slice<R, 4>(t.t11 + sc), v10 = load_slice<R, 4>(t.t10 + sc);
#pragma unroll
        for (int k = 0; k < 4; ++k)
          buf[k0 + k] = s.k00 * v00.v[k] + s.k01 * v01.v[k] + s.k11 * v11.v[k] + s.k10 * v10.v[k];
      }
    } else {
#pragma unroll
      for (int k = 0; k < kMaxSubChannels; ++k) {
        if (k < sub) {
          const int sc = gs * sub + k;
          buf[k] = s.k00 * t.t00[sc] + s.k01 * t.t01[sc] + s.k11 * t.t11[sc] + s.k10 * t.t10[sc];
        }
      }
    }
    for (int gi = 0; gi < groups; ++gi) {
      R tmp = R(0);
      if constexpr (SUB > 0) {
#pragma unroll
        for (int k0 = 0; k0 < SUB; k0 += 4) {
          const Slice<R, 4> r = load_slice<R, 4>(ref_px + gi * SUB + k0);
#pragma unroll
          for (int k = 0; k < 4; ++k) tmp += buf[k0 + k] * r.v[k];
        }
      } else {
#pragma unroll
        for (int k = 0; k < kMaxSubChannels; ++k)
          if (k < sub) tmp += buf[k] * ref_px[gi * sub + k];
      }
      if (best < tmp) {
        best = tmp;
        gi_out = gi;
        gs_out = gs;
      }
    }
  }
  return best;
}

template <typename R, int REDUCE, int SUB>
__global__ __launch_bounds__(kBlock) void v3_forward_kernel(const Args<R> a) {
  const int C = (int)a.C, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW;
  const int groups = a.groups, sub = C / groups;
  const int64_t total = a.voxels();
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * kBlock) {
    const Voxel<R> v = locate(a, i);
    const R *ref_px = a.ref + v.pix * C;
    R acc = REDUCE == 0 ? R(0) : Limits<R>::min_positive();
    int used = 0, wn = -1, wgi = -1, wgs = -1;
    for (int n = 0; n < N; ++n) {
      Sample<R> s;
      const int64_t cam = (int64_t)v.b * N + n;
      project(a.Rs + cam * 9, a.Ts + cam * 3, v.ref_w, v.ref_h, v.depth, a.half, srcH, srcW, s);
      if (s.state != 2) continue;
      const Taps<R> t = taps_of(a.src, s, cam, C, srcH, srcW);
      int gi = -1, gs = -1;
      if (REDUCE == 0) {
        acc += best_pair<R, SUB>(s, t, ref_px, groups, sub, Limits<R>::min_positive(), gi, gs);
        ++used;
      } else {
        const R best = best_pair<R, SUB>(s, t, ref_px, groups, sub, acc, gi, gs);
        if (gi >= 0) {
          acc = best;
          wn = n, wgi = gi, wgs = gs;
        }
      }
    }
    if (REDUCE == 0) {
      a.mask[i] = used;
      a.cost[i] = used > 0 ? acc / static_cast<R>(used) : R(0);
    } else {
      a.mask[i * 3] = wn, a.mask[i * 3 + 1] = wgi, a.mask[i * 3 + 2] = wgs;
      a.cost[i] = wn >= 0 ? acc : R(0);
    }
  }
}

// Thread -> voxel mapping of the gradient: the 64 lanes of a wave take 64 consecutive PIXELS
// at one depth, the four waves of a workgroup four consecutive depths, and the workgroup walks
// its segment of the depth range.  With the lanes along the depth axis (the reference's
// order) all lanes of an atomic instruction add into the same few texels of src_grad;
// neighbouring pixels hit neighbouring texels instead, and the rows of the pixel-owned
// gradients (ref_grad, base-plane gradient: all D voxels of a pixel add into the same row)
// are accumulated in LDS (ds_add) over the whole depth segment and leave as one global
// atomic per element and workgroup.  lds_rows = 0 selects plain global atomics (rows that do
// not fit).  What bounds the kernel either way is the number of source-gradient atomics, four
// taps times the channels of a group per (voxel, view), one element each: 10.6 ms for the
// gradient of the MVSNet-stage tensors (11.1 ms in the reference's order); the tiled kernels,
// which merge them in registers and LDS first, take 0.5 ms for the shapes they cover.
constexpr int kV3Pixels = 64, kV3Depths = kBlock / kV3Pixels;
template <typename R, int REDUCE, int SUB>
__global__ __launch_bounds__(kBlock) void v3_backward_kernel(const Args<R> a, int lds_rows,
                                                             int nsplit, int seg) {
  extern __shared__ __align__(16) unsigned char v3_smem[];
  R *rows = reinterpret_cast<R *>(v3_smem);  // [64][C + 1]: ref_grad row, depth gradient
  const int C = (int)a.C, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW, D = (int)a.D;
  const int groups = a.groups, sub = C / groups;
  const int64_t pixels = a.pixels();
  const int64_t row_step = (int64_t)srcW * C;
  const int RW = C + 1;
  const int64_t group = (int64_t)blockIdx.x / nsplit;
  const int split = (int)((int64_t)blockIdx.x - group * nsplit);
  const int64_t pix0 = group * kV3Pixels;
  const int lane_px = threadIdx.x % kV3Pixels, dw = threadIdx.x / kV3Pixels;
  const int64_t pix = pix0 + lane_px;
  const int d_lo = split * seg, d_hi = min(D, d_lo + seg);
  if (lds_rows > 0) {
    for (int k = threadIdx.x; k < kV3Pixels * RW; k += kBlock) rows[k] = R(0);
    __syncthreads();
  }
  for (int d = d_lo + dw; d < d_hi; d += kV3Depths) {
    if (pix >= pixels) break;
    const int64_t i = pix * D + d;
    const int32_t *m = a.mask_in + (REDUCE == 0 ? i : i * 3);
    const int32_t m0 = m[0];
    if (REDUCE == 0 ? (m0 > 0) : (m0 >= 0)) {
      const Voxel<R> v = locate(a, i);
      const R *ref_px = a.ref + v.pix * C;
      R *ref_lds = rows + lane_px * RW;         // (kept apart from the global row, so that
      R *ref_glb = a.ref_grad + v.pix * C;      //  the LDS adds compile to LDS instructions)
      // :426 cost_grad / (T)mask for the mean; the MIN gradient takes cost_grad as is (:621)
      const R cg = REDUCE == 0 ? a.cost_grad[i] / static_cast<R>(m0) : a.cost_grad[i];
      R depth_grad = R(0);
      const int n_lo = REDUCE == 0 ? 0 : m0, n_hi = REDUCE == 0 ? N : m0 + 1;
      for (int n = n_lo; n < n_hi && n < N; ++n) {
        Sample<R> s;
        const int64_t cam = (int64_t)v.b * N + n;
        project(a.Rs + cam * 9, a.Ts + cam * 3, v.ref_w, v.ref_h, v.depth, a.half, srcH, srcW, s);
        // A winner that is not accepted any more (inputs changed since the forward pass) is
        // skipped; the reference would read and write out of bounds (:593-595).
        if (s.state != 2) continue;
        const Taps<R> t = taps_of(a.src, s, cam, C, srcH, srcW);
        int gi = -1, gs = -1;
        if (REDUCE == 0) {
          best_pair<R, SUB>(s, t, ref_px, groups, sub, Limits<R>::min_positive(), gi, gs);
          // no pair above the seed: the reference indexes group -1 here (:495-496)
          if (gi < 0) continue;
        } else {
          gi = m[1], gs = m[2];
          if (gi < 0 || gi >= groups || gs < 0 || gs >= groups) continue;
        }
        R *g00 = a.src_grad + (t.t00 - a.src);
        R h_grad = R(0), w_grad = R(0);
        for (int k = 0; k < sub; ++k) {
          const int rc = gi * sub + k, cc = gs * sub + k;
          const R v00 = t.t00[cc], v01 = t.t01[cc], v11 = t.t11[cc], v10 = t.t10[cc];
          const R smp = s.k00 * v00 + s.k01 * v01 + s.k11 * v11 + s.k10 * v10;
          if (lds_rows > 0)
            __hip_atomic_fetch_add(ref_lds + rc, cg * smp, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_WORKGROUP);
          else
            atomic_add(ref_glb + rc, cg * smp);
          const R bg = cg * ref_px[rc];
          atomic_add(g00 + cc, bg * s.k00);
          atomic_add(g00 + C + cc, bg * s.k01);
          atomic_add(g00 + C + row_step + cc, bg * s.k11);
          atomic_add(g00 + row_step + cc, bg * s.k10);
          const R t1 = v11 - v10 - v01 + v00;
          h_grad += bg * (t1 * s.dw + v10 - v00);
          w_grad += bg * (t1 * s.dh + v01 - v00);
        }
        depth_grad += depth_chain(s, h_grad, w_grad);
      }
      if (lds_rows > 0)
        __hip_atomic_fetch_add(ref_lds + C, depth_grad, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
      else
        atomic_add(a.depth_grad + v.pix, depth_grad);
    }
  }
  if (lds_rows > 0) {
    __syncthreads();
    for (int k = threadIdx.x; k < kV3Pixels * RW; k += kBlock) {
      const int r = k / RW, c = k - r * RW;
      const R val = rows[k];
      if (val != R(0) && pix0 + r < pixels) {
        if (c < C)
          atomic_add(a.ref_grad + (pix0 + r) * C + c, val);
        else
          atomic_add(a.depth_grad + pix0 + r, val);
      }
    }
  }
}

// ---- FeatureAggregate --------------------------------------------------------------------
template <typename R, int VEC>
__global__ __launch_bounds__(kBlock) void feature_forward_kernel(const Args<R> a) {
  const int C = (int)a.C, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW;
  const int slices = C / VEC;
  const int64_t total = a.voxels() * N * slices;
  for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * kBlock) {
    const int64_t row = e / slices;  // (voxel, view)
    const int c0 = (int)(e - row * slices) * VEC;
    const int64_t i = row / N;
    const int n = (int)(row - i * N);
    const Voxel<R> v = locate(a, i);
    Sample<R> s;
    const int64_t cam = (int64_t)v.b * N + n;
    project(a.Rs + cam * 9, a.Ts + cam * 3, v.ref_w, v.ref_h, v.depth, a.half, srcH, srcW, s);
    Slice<R, VEC> out;
    if (s.state == 2) {
      const Taps<R> t = taps_of(a.src, s, cam, C, srcH, srcW);
      const Slice<R, VEC> v00 = load_slice<R, VEC>(t.t00 + c0), v01 = load_slice<R, VEC>(t.t01 + c0),
                          v11 = load_slice<R, VEC>(t.t11 + c0), v10 = load_slice<R, VEC>(t.t10 + c0);
#pragma unroll
      for (int k = 0; k < VEC; ++k)
        out.v[k] = s.k00 * v00.v[k] + s.k01 * v01.v[k] + s.k11 * v11.v[k] + s.k10 * v10.v[k];
    } else {
#pragma unroll
      for (int k = 0; k < VEC; ++k) out.v[k] = R(0);
    }
    store_slice<R, VEC>(a.cost + row * C + c0, out);
    if (c0 == 0) a.mask[row] = s.state == 2 ? 1 : 0;
  }
}

template <typename R, int VEC>
__global__ __launch_bounds__(kBlock) void feature_backward_kernel(const Args<R> a) {
  const int C = (int)a.C, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW;
  const int slices = C / VEC;
  const int64_t total = a.voxels() * N * slices;
  const int64_t row_step = (int64_t)srcW * C;
  for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * kBlock) {
    const int64_t row = e / slices;
    const int c0 = (int)(e - row * slices) * VEC;
    if (a.mask_in[row] == 0) continue;  // :261-263
    const int64_t i = row / N;
    const int n = (int)(row - i * N);
    const Voxel<R> v = locate(a, i);
    Sample<R> s;
    const int64_t cam = (int64_t)v.b * N + n;
    project(a.Rs + cam * 9, a.Ts + cam * 3, v.ref_w, v.ref_h, v.depth, a.half, srcH, srcW, s);
    // the reference trusts the mask (:271, :284-285); a sample that is not accepted any more
    // is skipped instead of read out of bounds
    if (s.state != 2) continue;
    const Taps<R> t = taps_of(a.src, s, cam, C, srcH, srcW);
    R *g00 = a.src_grad + (t.t00 - a.src) + c0;
    const Slice<R, VEC> g = load_slice<R, VEC>(a.cost_grad + row * C + c0);
    const Slice<R, VEC> v00 = load_slice<R, VEC>(t.t00 + c0), v01 = load_slice<R, VEC>(t.t01 + c0),
                        v11 = load_slice<R, VEC>(t.t11 + c0), v10 = load_slice<R, VEC>(t.t10 + c0);
    R h_grad = R(0), w_grad = R(0);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      atomic_add(g00 + k, g.v[k] * s.k00);
      atomic_add(g00 + C + k, g.v[k] * s.k01);
      atomic_add(g00 + C + row_step + k, g.v[k] * s.k11);
      atomic_add(g00 + row_step + k, g.v[k] * s.k10);
      const R t1 = v11.v[k] - v10.v[k] - v01.v[k] + v00.v[k];
      h_grad += g.v[k] * (t1 * s.dw + v10.v[k] - v00.v[k]);
      w_grad += g.v[k] * (t1 * s.dh + v01.v[k] - v00.v[k]);
    }
    atomic_add(a.depth_grad + v.pix, depth_chain(s, h_grad, w_grad));
  }
}

template <typename R>
bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

}  // namespace

// 4 or 8 when a channel group is that many floats and every row starts 16-byte aligned
// (the pair search then uses 16-byte loads), 0 otherwise.
template <typename S>
int v3_vector_width(const Args<S> &a) {
  const int64_t sub = a.C / a.groups;
  if (!std::is_same<S, float>::value || (sub != 4 && sub != 8)) return 0;
  if (!aligned16<S>(a.src) || !aligned16<S>(a.ref)) return 0;
  return (int)sub;
}

template <typename S>
hipError_t launch_v3_forward(const Args<S> &a, hipStream_t stream) {
  const int64_t total = a.voxels();
  if (total == 0) return hipSuccess;
  const int grid = grid_for(total, kBlock);
  const int sub = v3_vector_width(a);
#define CHOP_V3_FWD(RED, SUB) v3_forward_kernel<S, RED, SUB><<<grid, kBlock, 0, stream>>>(a)
  if (a.reduce == 0) {
    if (sub == 8) CHOP_V3_FWD(0, 8); else if (sub == 4) CHOP_V3_FWD(0, 4); else CHOP_V3_FWD(0, 0);
  } else {
    if (sub == 8) CHOP_V3_FWD(1, 8); else if (sub == 4) CHOP_V3_FWD(1, 4); else CHOP_V3_FWD(1, 0);
  }
#undef CHOP_V3_FWD
  return hipGetLastError();
}

template <typename S>
hipError_t launch_v3_backward(const Args<S> &a, hipStream_t stream) {
  hipError_t err;
  ZeroRanges zero;  // one launch
  zero.add(a.ref_grad, (size_t)(a.pixels() * a.C) * sizeof(S));
  zero.add(a.src_grad, (size_t)(a.B * a.N * a.srcH * a.srcW * a.C) * sizeof(S));
  zero.add(a.depth_grad, (size_t)a.pixels() * sizeof(S));
  if ((err = zero.launch(stream)) != hipSuccess) return err;
  const int64_t total = a.voxels();
  if (total == 0 || a.C == 0) return hipSuccess;
  const int sub = v3_vector_width(a);
  // workgroups: groups of 64 pixels, times enough depth segments to give every SIMD a few
  // waves (whole rounds of the four depths a workgroup covers at a time)
  const int64_t pixel_groups = (a.pixels() + kV3Pixels - 1) / kV3Pixels;
  int64_t nsplit = (256 * 4 * 2 + pixel_groups - 1) / pixel_groups;
  const int64_t rounds = (a.D + kV3Depths - 1) / kV3Depths;
  if (nsplit > rounds) nsplit = rounds;
  if (nsplit < 1) nsplit = 1;
  const int seg = (int)((rounds + nsplit - 1) / nsplit) * kV3Depths;
  nsplit = (a.D + seg - 1) / seg;
  if (pixel_groups * nsplit >= (int64_t)1 << 31) return hipErrorInvalidValue;
  const dim3 grid((unsigned)(pixel_groups * nsplit));
  // the rows of the workgroup's pixels in LDS
  int lds_rows = kV3Pixels;
  size_t smem = (size_t)lds_rows * (size_t)(a.C + 1) * sizeof(S);
  if (smem > 32 * 1024) lds_rows = 0, smem = 0;
#define CHOP_V3_BWD(RED, SUB) \
  v3_backward_kernel<S, RED, SUB><<<grid, kBlock, smem, stream>>>(a, lds_rows, (int)nsplit, seg)
  if (a.reduce == 0) {
    if (sub == 8) CHOP_V3_BWD(0, 8); else if (sub == 4) CHOP_V3_BWD(0, 4); else CHOP_V3_BWD(0, 0);
  } else {
    CHOP_V3_BWD(1, 0);  // the winner comes from the mask: no pair search
  }
#undef CHOP_V3_BWD
  return hipGetLastError();
}

template <typename S>
hipError_t launch_feature_forward(const Args<S> &a, hipStream_t stream) {
  constexpr int kVec = 16 / (int)sizeof(S);
  const bool wide = a.C % kVec == 0 && aligned16<S>(a.src) && aligned16<S>(a.cost);
  const int64_t total = a.voxels() * a.N * (wide ? a.C / kVec : a.C);
  if (total == 0) return hipSuccess;
  const int grid = grid_for(total, kBlock);
  if (wide)
    feature_forward_kernel<S, kVec><<<grid, kBlock, 0, stream>>>(a);
  else
    feature_forward_kernel<S, 1><<<grid, kBlock, 0, stream>>>(a);
  return hipGetLastError();
}

template <typename S>
hipError_t launch_feature_backward(const Args<S> &a, hipStream_t stream) {
  hipError_t err;
  ZeroRanges zero;  // one launch
  zero.add(a.src_grad, (size_t)(a.B * a.N * a.srcH * a.srcW * a.C) * sizeof(S));
  zero.add(a.depth_grad, (size_t)a.pixels() * sizeof(S));
  if ((err = zero.launch(stream)) != hipSuccess) return err;
  constexpr int kVec = 16 / (int)sizeof(S);
  const bool wide = a.C % kVec == 0 && aligned16<S>(a.src) && aligned16<S>(a.cost_grad);
  const int64_t total = a.voxels() * a.N * (wide ? a.C / kVec : a.C);
  if (total == 0) return hipSuccess;
  const int grid = grid_for(total, kBlock);
  if (wide)
    feature_backward_kernel<S, kVec><<<grid, kBlock, 0, stream>>>(a);
  else
    feature_backward_kernel<S, 1><<<grid, kBlock, 0, stream>>>(a);
  return hipGetLastError();
}

#define CHOP_INSTANTIATE(S)                                                       \
  template hipError_t launch_v3_forward<S>(const Args<S> &, hipStream_t);         \
  template hipError_t launch_v3_backward<S>(const Args<S> &, hipStream_t);        \
  template hipError_t launch_feature_forward<S>(const Args<S> &, hipStream_t);    \
  template hipError_t launch_feature_backward<S>(const Args<S> &, hipStream_t);
CHOP_INSTANTIATE(float)
CHOP_INSTANTIATE(double)
#undef CHOP_INSTANTIATE

}  // namespace chop
