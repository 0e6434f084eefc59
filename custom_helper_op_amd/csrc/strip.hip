// Strip kernels: the wave-per-pixel-strip decomposition for every shape the tiled kernels do
// not take -- float64 (the element type of the reference's own tests), channel counts that
// are not 4 x a power of two (the reference tests use 3, 5 and 9), any number of views -- for
// CostVolume, CostVolumeV2, CostAggregate (both reduces) and FeatureAggregate, all four storage
// types, up to 64 channels; and for the gradient of CostVolumeV3 in float and double with any
// group width (the lanes of a pixel find the view's best group pair again through LDS, then
// only the winning source group's lanes add into their taps).
//
// A workgroup is one wavefront.  It owns 64/LPP consecutive pixels (LPP = the power of two
// >= C: one lane per channel, so a tap read or a cost-row write of a pixel is one contiguous
// C-element segment) and one segment of the depth hypotheses, walked in chunks of kDB depths
// with the views as the middle loop:
//   phase 1  the lanes of a pixel reproject the chunk's depths into a group of views (lane
//            -> (view of the group, depth): a pixel of 32 lanes serves four views at once; the
//            bit-exact code of warp.h) and leave one record per (view, pixel, depth) in LDS;
//   phase 2  view by view, every lane walks the chunk's depths for its channel; the four taps
//            stay in registers while consecutive depths fall into the same texel cell.
// Forward: the arithmetic is the reference's literal operand order, every operation rounded
// separately (cost_volume_kernels_gpu.cu.cc:33-228, cost_volume_kernels_gpu_v2.cu.cc:33-235),
// views and channels summed in the reference's order, so float and double results are
// bit-identical to a plain IEEE CPU evaluation, as with the general kernels.
// Backward (:342-577, v2 :349-601): ref_grad and the base-plane gradient are pixel-owned and
// stay in registers; the source-gradient contributions of a run of depths that share a cell
// are merged in registers and leave as one atomic add per tap and channel when the cell
// changes (the reference issues one per voxel) -- a run that is still open at the end of a
// chunk waits in LDS for the view's turn in the next chunk; the per-voxel depth gradient is
// summed over the pixel's lanes in registers and stored once.  Wide pixels in double (16 lanes
// or more: at most four pixels per wave, whose atomics would each carry one pixel's channels)
// put a small write-back cache of texels in LDS between the runs and memory: consecutive runs
// of a pixel and its neighbours hit the same texels, and a texel leaves as one atomic per
// channel when another texel needs its slot; with the cache a run ends with its chunk (it is
// not carried), which leaves LDS for a fourth wave per SIMD.
#include <type_traits>

#include "internal.h"

namespace chop {

namespace {

constexpr int kDB = 8;  // depths per chunk (16 measured slower everywhere: registers)

struct StripGeom {
  int lpp_shift;        // log2(LPP)
  int nseg, seg;        // depth segments, depths per segment (a multiple of kDB)
  int vg;               // views reprojected together: min(N, max(1, LPP / kDB))
  int carry;            // backward: open runs survive the end of a chunk (in LDS)
  int cache;            // backward: a texel cache in LDS between the runs and memory
  int pair_bytes;       // backward of CostVolumeV3: LDS of the group-pair search (0 otherwise)
  int64_t tiles;        // ceil(B*H*W / PPW)
};

__device__ __forceinline__ void strip_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// 1 / x to within an ulp or two, for the backward's factors (a full IEEE division costs about
// ten instructions in float and fifty in double; the gradients are compared at 1e-4).
__device__ __forceinline__ float quick_recip(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ double quick_recip(double x) {
  double r = __builtin_amdgcn_rcp(x);
  r = __builtin_fma(__builtin_fma(-x, r, 1.0), r, r);
  return __builtin_fma(__builtin_fma(-x, r, 1.0), r, r);
}

// a * b + c in one rounding: the backward's arithmetic (gradients are compared at 1e-4; with
// contraction off for the whole library a plain a * b + c is two instructions)
__device__ __forceinline__ float mad(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double mad(double a, double b, double c) { return __builtin_fma(a, b, c); }

// Sum over the 2^shift consecutive lanes of a pixel, left in every one of them.
template <typename R>
__device__ __forceinline__ R pixel_sum(R v, int shift) {
  for (int s = 0; s < shift; ++s) v += __shfl_xor(v, 1 << s, 64);
  return v;
}

template <typename R>
struct StripPixel {
  int64_t pix;
  int b;
  R ref_w, ref_h;
  bool ok;
};

template <typename S>
__device__ __forceinline__ StripPixel<typename Storage<S>::Real> strip_pixel(const Args<S> &a,
                                                                              int64_t pix) {
  using R = typename Storage<S>::Real;
  StripPixel<R> px;
  const int64_t npix = a.pixels();
  px.ok = pix < npix;
  px.pix = px.ok ? pix : npix - 1;  // clamp: loads stay in range, stores are predicated
  const int64_t row = px.pix / a.W;
  const int w = (int)(px.pix - row * a.W);
  px.b = (int)(row / a.H);
  const int h = (int)(row - (int64_t)px.b * a.H);
  px.ref_w = static_cast<R>(w) + a.half;
  px.ref_h = static_cast<R>(h) + a.half;
  return px;
}

// LDS of one wavefront: kDB records per (view of the group, pixel); a record is addressed
// [field][(view*PPW + pixel)*kDB + j].
template <typename R>
struct StripRecords {
  R *f;      // NF fields of vg*PPW*kDB values each
  int *off;  // tap offset inside the view, -1: nothing to do
  int *key;  // backward: the cell as (row << 16) | column
  int stride;
  __device__ __forceinline__ R &at(int field, int idx) { return f[field * stride + idx]; }
};

template <typename R, int NF>
__device__ __forceinline__ StripRecords<R> strip_records(unsigned char *smem, int records) {
  StripRecords<R> r;
  r.stride = records;
  r.f = reinterpret_cast<R *>(smem);
  r.off = reinterpret_cast<int *>(smem + (size_t)NF * r.stride * sizeof(R));
  r.key = r.off + records;
  return r;
}

// `records` = vg * PPW * (depths per chunk), then 64 values of staging
template <typename R>
constexpr size_t strip_lds_bytes(int nf, int records, int nints = 1) {
  return (size_t)records * (nf * sizeof(R) + nints * sizeof(int)) + 64 * sizeof(R);
}

// Runs that are open at the end of a chunk: per view and lane four tap sums, the tap offset
// and the cell.
template <typename S>
constexpr size_t strip_run_bytes(int64_t N) {
  return (size_t)N * 64 * (4 * sizeof(typename Storage<S>::Real) + 2 * sizeof(int));
}

// Texel cache of the backward kernel: per view kCacheRows x kCacheCols slots addressed by the
// low bits of the texel coordinates (direct-mapped), one value per lane of a pixel and a tag
// (the texel's index over all images of the call, -1: empty) per slot.  Two rows by four
// columns hold what a pixel and its neighbours in the strip work on at any time: the cells
// of consecutive runs share two of their four texels, and a slot is needed again only two
// rows or four columns further along the walk.
constexpr int kCacheRows = 2, kCacheCols = 4, kCacheSlots = kCacheRows * kCacheCols;
template <typename R>
constexpr size_t strip_cache_bytes(int64_t N, int lpp) {
  return (size_t)N * kCacheSlots * ((size_t)lpp * sizeof(R) + sizeof(int));
}

// ------------------------------------------------------------------------------------------
// Forward
// ------------------------------------------------------------------------------------------
template <typename S, int CORR, int REDUCE>
__global__ __launch_bounds__(64) void strip_forward_kernel(const Args<S> a, const StripGeom g) {
  using R = typename Storage<S>::Real;
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x, lpp = 1 << g.lpp_shift, ppw = 64 >> g.lpp_shift;
  const int p = lane >> g.lpp_shift, cl = lane & (lpp - 1);
  const int64_t tile = (int64_t)blockIdx.x / g.nseg;
  const int segi = (int)((int64_t)blockIdx.x - tile * g.nseg);
  const int C = (int)a.C, D = (int)a.D, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW;
  constexpr bool AGG = CORR == 2;   // CostAggregate: one value per voxel
  constexpr bool FEAT = CORR == 4;  // FeatureAggregate: the samples themselves, a row per view
  const int OC = CORR == 1 ? a.groups : AGG ? 1 : C;
  const int sub = CORR == 1 ? C / a.groups : 1;
  const int d_lo = segi * g.seg, d_hi = min(D, d_lo + g.seg);
  const StripPixel<R> px = strip_pixel(a, tile * ppw + p);
  const bool ch_ok = cl < C, out_ok = px.ok && cl < OC;
  const R ref_c = ch_ok && !FEAT ? Storage<S>::load(a.ref + px.pix * C + cl) : R(0);
  const R base = a.depth_grid ? R(0) : a.base_plane[px.pix];
  const bool fill = a.default_cost != nullptr;  // the cost-map layers' default for empty voxels
  const R dflt = fill ? *a.default_cost : R(0);
  const int64_t row_step = (int64_t)srcW * C;
  StripRecords<R> rec = strip_records<R, 4>(smem, ppw * g.vg * kDB);
  // group correlation: the products of a pixel's channels
  R *s_prod = reinterpret_cast<R *>(smem + strip_lds_bytes<R>(4, ppw * g.vg * kDB)) - 64;
  // CostAggregate: the chunk's squared differences, one row of 64 lanes per depth.  Lane
  // (jj mod LPP) of a pixel owns voxel (pixel, d0 + jj): it adds the row up in channel order,
  // which is the order of the reference's scalar loop (cost_aggregate_kernels_gpu.cu.cc:
  // 108-113, :206-216), so the sums and the winning views are the oracle's to the bit.
  R *s_rows = s_prod + 64;

  for (int d0 = d_lo; d0 < d_hi; d0 += kDB) {
    R acc[kDB];
    int arg[kDB], kcnt[kDB];
#pragma unroll
    for (int jj = 0; jj < kDB; ++jj) {
      acc[jj] = REDUCE == 0 ? R(0) : (CORR == 1 ? Limits<R>::min_positive() : Limits<R>::max());
      arg[jj] = -1;
      kcnt[jj] = 0;
    }
    for (int n0 = 0; n0 < N; n0 += g.vg) {
      const int nv = min(g.vg, N - n0);
      strip_sync();  // the records of the views before have been read
      for (int item = cl; item < nv * kDB; item += lpp) {
        const int nl = item / kDB, j = item - nl * kDB;
        const int64_t cam = (int64_t)px.b * N + n0 + nl;
        const int d = d0 + j;
        int off = -1;
        Sample<R> s;
        s.k00 = s.k01 = s.k11 = s.k10 = R(0);
        if (d < d_hi) {
          const R depth = a.depth_grid ? a.depth_grid[px.pix * D + d]
                                       : base + a.offsets[(int64_t)px.b * D + d];
          project(a.Rs + cam * 9, a.Ts + cam * 3, px.ref_w, px.ref_h, depth, a.half, srcH, srcW, s);
          if (s.state == 2) off = (s.fh * srcW + s.fw) * C;
        }
        const int r = (nl * ppw + p) * kDB + j;
        rec.off[r] = off;
        rec.at(0, r) = s.k00;
        rec.at(1, r) = s.k01;
        rec.at(2, r) = s.k11;
        rec.at(3, r) = s.k10;
      }
      strip_sync();
      for (int nl = 0; nl < nv; ++nl) {
        const int n = n0 + nl;
        const int ridx = (nl * ppw + p) * kDB;
        const int64_t cam = (int64_t)px.b * N + n;
        const S *view = a.src + cam * srcH * srcW * C + (ch_ok ? cl : 0);
        int cur = -1;
        R v00 = R(0), v01 = R(0), v11 = R(0), v10 = R(0);
#pragma unroll
        for (int jj = 0; jj < kDB; ++jj) {
          const int off = rec.off[ridx + jj];
          if constexpr (FEAT) {
            // zeros and a 0 in the mask for a view that is not accepted
            // (feature_aggregate_kernels_gpu.cu.cc:114-118)
            if (off < 0) {
              const int64_t row = (px.pix * D + d0 + jj) * N + n;
              if (d0 + jj < d_hi && px.ok) {
                if (ch_ok) Storage<S>::store(a.cost + row * C + cl, R(0));
                if (cl == 0) a.mask[row] = 0;
              }
            }
          }
          if (off < 0) continue;
          if (off != cur) {
            cur = off;
            const S *q = view + off;
            v00 = Storage<S>::load(q), v01 = Storage<S>::load(q + C);
            v11 = Storage<S>::load(q + C + row_step), v10 = Storage<S>::load(q + row_step);
          }
          const R smp = rec.at(0, ridx + jj) * v00 + rec.at(1, ridx + jj) * v01 +
                        rec.at(2, ridx + jj) * v11 + rec.at(3, ridx + jj) * v10;
          if constexpr (FEAT) {
            const int64_t row = (px.pix * D + d0 + jj) * N + n;
            if (px.ok) {  // (an accepted record implies d0 + jj < d_hi)
              if (ch_ok) Storage<S>::store(a.cost + row * C + cl, smp);
              if (cl == 0) a.mask[row] = 1;
            }
            continue;
          }
          R val;
          if (CORR != 1) {
            const R diff = smp - ref_c;
            val = diff * diff;
            if constexpr (AGG) {
              s_rows[jj * 64 + lane] = val;
              continue;
            }
          } else {
            // the group's products, added up from zero in channel order by the group's lane
            s_prod[lane] = smp * ref_c;
            strip_sync();
            val = R(0);
            if (cl < OC)
              for (int c = 0; c < sub; ++c) val += s_prod[p * lpp + cl * sub + c];
            strip_sync();
          }
          if (REDUCE == 0) {
            acc[jj] += val;
          } else if (CORR == 1 ? (acc[jj] < val) : (acc[jj] > val)) {
            acc[jj] = val;
            arg[jj] = n;
          }
          ++kcnt[jj];
        }
        if constexpr (AGG) {
          strip_sync();  // the rows are written
          // the owners work side by side: lane cl owns depths cl, cl + LPP, ... of its pixel
          // (acc / kcnt / arg are indexed by k, the k-th depth a lane owns)
#pragma unroll
          for (int k = 0; k < kDB; ++k) {
            const int jj = cl + k * lpp;
            if (jj >= kDB || rec.off[ridx + jj] < 0) continue;
            const R *row = s_rows + jj * 64 + p * lpp;
            // eight LDS reads in flight, then eight additions in channel order
            R sum = REDUCE == 0 ? acc[k] : R(0);
            for (int c0 = 0; c0 < C; c0 += 8) {
              R v[8];
#pragma unroll
              for (int u = 0; u < 8; ++u) v[u] = row[min(c0 + u, C - 1)];
#pragma unroll
              for (int u = 0; u < 8; ++u)
                if (c0 + u < C) sum += v[u];
            }
            if (REDUCE == 0) {
              acc[k] = sum;
              ++kcnt[k];
            } else if (acc[k] > sum) {
              acc[k] = sum, arg[k] = n;  // strict: the earliest view keeps a tie
            }
          }
          strip_sync();  // ... and read, before the next view overwrites them
        }
      }
    }  // group of views
    if constexpr (FEAT) continue;  // every row has been stored
    if constexpr (AGG) {
#pragma unroll
      for (int k = 0; k < kDB; ++k) {
        const int jj = cl + k * lpp, d = d0 + jj;
        if (jj >= kDB || d >= d_hi || !px.ok) continue;
        const int64_t i = px.pix * D + d;
        const bool any = REDUCE == 0 ? kcnt[k] > 0 : arg[k] >= 0;
        // :118-123 cost / (T)(used * channels), :222-227 cost / (T)channels
        R out = REDUCE == 0 ? acc[k] / static_cast<R>((int64_t)kcnt[k] * C)
                            : acc[k] / static_cast<R>(C);
        if (!any) out = fill ? dflt : R(0);
        a.mask[i] = REDUCE == 0 ? kcnt[k] : arg[k];
        Storage<S>::store(a.cost + i, out);
      }
      continue;
    }
#pragma unroll
    for (int jj = 0; jj < kDB; ++jj) {
      const int d = d0 + jj;
      if (d >= d_hi) break;
      const int64_t i = px.pix * D + d;
      if (REDUCE == 0) {
        // the mean: halving and quartering are exact, so only other counts pay for a division
        if (kcnt[jj] == 2)
          acc[jj] = acc[jj] * R(0.5);
        else if (kcnt[jj] == 4)
          acc[jj] = acc[jj] * R(0.25);
        else if (kcnt[jj] > 2)
          acc[jj] = acc[jj] / static_cast<R>(kcnt[jj]);
        if (px.ok && cl == 0) a.mask[i] = kcnt[jj];
      } else if (out_ok) {
        a.mask[i * OC + cl] = arg[jj];
      }
      if (fill && (REDUCE == 0 ? kcnt[jj] == 0 : arg[jj] < 0)) acc[jj] = dflt;
      if (out_ok) Storage<S>::store(a.cost + i * OC + cl, acc[jj]);
    }
  }
}

// ------------------------------------------------------------------------------------------
// Backward
// ------------------------------------------------------------------------------------------
// W4: compiled for four waves per SIMD.  In double the kernel needs 128-168 registers as
// written; held to 128 (20-56 bytes of scratch per lane for most terms and reduces, up to 160
// for the group correlation's maximum) it runs four waves instead of three wherever LDS lets
// it, which is worth 12-22 % with wide pixels (see strip_geometry).  The gradients of a mean
// take that form always (130 registers as written; narrow pixels gain 4-6 %), those of a
// minimum / maximum only with wide pixels (3 channels in double: 6 % slower with the scratch
// and nothing to gain, LDS holds such launches to ten workgroups per compute unit).  Float
// and 16-bit storage stay below 128 registers by themselves.

template <typename S, int CORR, int REDUCE, bool W4 = false>
__global__ __launch_bounds__(64, W4 ? 4 : 1) void strip_backward_kernel(const Args<S> a, const StripGeom g) {
  using R = typename Storage<S>::Real;
  using Acc = typename std::conditional<sizeof(S) == 2, float, S>::type;
  extern __shared__ __align__(16) unsigned char smem[];
  Acc *ref_grad = sizeof(S) == 2 ? (Acc *)a.ref_grad_acc : (Acc *)a.ref_grad;
  Acc *src_grad = sizeof(S) == 2 ? (Acc *)a.src_grad_acc : (Acc *)a.src_grad;
  const int lane = threadIdx.x, lpp = 1 << g.lpp_shift, ppw = 64 >> g.lpp_shift;
  const int p = lane >> g.lpp_shift, cl = lane & (lpp - 1);
  const int64_t tile = (int64_t)blockIdx.x / g.nseg;
  const int segi = (int)((int64_t)blockIdx.x - tile * g.nseg);
  const int C = (int)a.C, D = (int)a.D, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW;
  constexpr bool AGG = CORR == 2;   // CostAggregate: one upstream value per voxel
  constexpr bool FEAT = CORR == 4;  // FeatureAggregate: an upstream row and a mask entry per view
  constexpr bool PAIR = CORR == 3;  // CostVolumeV3: one value per voxel, from the best group pair
  const int OC = CORR == 1 ? a.groups : (AGG || PAIR) ? 1 : C;
  const int MS = PAIR && REDUCE != 0 ? 3 : OC;  // mask entries per voxel (V3 MIN: view, two groups)
  const int sub = (CORR == 1 || PAIR) ? C / a.groups : 1;
  const int G = PAIR ? a.groups : 1;
  const int d_lo = segi * g.seg, d_hi = min(D, d_lo + g.seg);
  const StripPixel<R> px = strip_pixel(a, tile * ppw + p);
  const bool ch_ok = cl < C && px.ok;
  const int oc = CORR == 1 ? (ch_ok ? cl / sub : 0) : (AGG || PAIR) ? 0 : (ch_ok ? cl : 0);
  const R ref_c = ch_ok && !FEAT ? Storage<S>::load(a.ref + px.pix * C + cl) : R(0);
  const R base = a.depth_grid ? R(0) : a.base_plane[px.pix];
  // per-voxel hypotheses: always for the group correlation, never for the ops over a base
  // plane; the squared difference has them through the 16-bit entry points only (known at
  // compile time wherever possible: the per-voxel sums of a chunk are 16 registers in double)
  const bool per_voxel = CORR == 1 || (CORR == 0 && sizeof(S) == 2 && a.depth_grid != nullptr);
  const bool want_depth = a.depth_grad != nullptr;
  const int64_t row_step = (int64_t)srcW * C;
  // fields: the four weights, dh, dw, the two depth-chain factors, 1 / view count
  // (CostAggregate: 1 / (view count * channels), or 1 / channels for the MIN reduce)
  StripRecords<R> rec = strip_records<R, 9>(smem, ppw * g.vg * kDB);
  // open runs between two chunks: per view the cell and its four tap sums, one slot per lane
  // (a lane only ever reads its own slots back)
  R *s_run = reinterpret_cast<R *>(smem + strip_lds_bytes<R>(9, ppw * g.vg * kDB, 2));
  int *s_cur = reinterpret_cast<int *>(s_run + (size_t)N * 4 * 64);
  const bool carry = g.carry != 0;
  if (carry)
    for (int n = 0; n < N; ++n) s_cur[n * 64 + lane] = -1;
  int *s_ckey = s_cur + (size_t)N * 64;  // the carried runs' cells as (row << 16) | column
  // texel cache: values [view][slot][lane of the pixel], then the tags
  const bool cache = g.cache != 0;
  R *s_val = reinterpret_cast<R *>(reinterpret_cast<unsigned char *>(s_run) +
                                   (carry ? strip_run_bytes<S>(N) : 0));
  int *s_tag = reinterpret_cast<int *>(s_val + (size_t)N * kCacheSlots * lpp);
  if (cache)
    for (int k = lane; k < N * kCacheSlots; k += 64) s_tag[k] = -1;
  const unsigned long long pix_lanes = lpp == 64 ? ~0ull : ((1ull << lpp) - 1ull);
  // CostVolumeV3: the pixels' reference rows and the samples of the depth at hand
  R *s_ref = reinterpret_cast<R *>(reinterpret_cast<unsigned char *>(s_val) +
                                   (cache ? strip_cache_bytes<R>(N, lpp) : 0));
  R *s_smp = s_ref + 64;
  const int my_group = PAIR && ch_ok ? cl / sub : -1, my_k = PAIR && ch_ok ? cl - my_group * sub : 0;
  if constexpr (PAIR) s_ref[lane] = ref_c;
  const int64_t img_texels = (int64_t)srcH * srcW;
  R racc = R(0), dpart = R(0);

  for (int d0 = d_lo; d0 < d_hi; d0 += kDB) {
    R dvox[kDB];
#pragma unroll
    for (int jj = 0; jj < kDB; ++jj) dvox[jj] = R(0);
    // This lane's upstream gradients (and, for the MIN reduce, winners) of the chunk's depths,
    // requested together and ahead of the reprojection: fetched one by one where a depth
    // uses them, every depth of every wave waits for memory (the kernel spent two thirds of
    // its time in such waits).  They serve all views.
    R cgv[kDB];
    int win[REDUCE != 0 ? kDB : 1];
    int win_gi[PAIR && REDUCE != 0 ? kDB : 1], win_gs[PAIR && REDUCE != 0 ? kDB : 1];
    if constexpr (!FEAT) {
#pragma unroll
      for (int jj = 0; jj < kDB; ++jj) {
        const int64_t i = px.pix * D + min(d0 + jj, d_hi - 1);
        cgv[jj] = Storage<S>::load(a.cost_grad + i * OC + oc);
        if constexpr (REDUCE != 0) win[jj] = a.mask_in[i * MS + oc];
        if constexpr (PAIR && REDUCE != 0)
          win_gi[jj] = a.mask_in[i * MS + 1], win_gs[jj] = a.mask_in[i * MS + 2];
      }
    }
    for (int n0 = 0; n0 < N; n0 += g.vg) {
      const int nv = min(g.vg, N - n0);
      strip_sync();
      for (int item = cl; item < nv * kDB; item += lpp) {
        const int nl = item / kDB, j = item - nl * kDB;
        const int64_t cam = (int64_t)px.b * N + n0 + nl;
        const int ridx = (nl * ppw + p) * kDB;
        const int d = d0 + j;
        int off = -1;
        Sample<R> s;
        s.k00 = s.k01 = s.k11 = s.k10 = s.dh = s.dw = R(0);
        R fh = R(0), fw = R(0), cnt = R(1);
        // every load of this item goes out before the first test, so that the item waits for
        // memory once (mask, then depth, then camera, each behind a branch, were three waits)
        const int64_t i = px.pix * D + min(d, d_hi - 1);
        // FeatureAggregate: 1 / 0 per (voxel, view), :261-263
        const int32_t m0 = FEAT ? a.mask_in[i * N + n0 + nl] : a.mask_in[REDUCE == 0 ? i : i * MS];
        const R dval = per_voxel ? a.depth_grid[i] : a.offsets[(int64_t)px.b * D + min(d, d_hi - 1)];
        R Rm[9], Tv[3];
#pragma unroll
        for (int k = 0; k < 9; ++k) Rm[k] = a.Rs[cam * 9 + k];
#pragma unroll
        for (int k = 0; k < 3; ++k) Tv[k] = a.Ts[cam * 3 + k];
        if (d < d_hi && px.ok) {
          // MEAN skips a voxel no view reached (:367), MIN one whose first entry is negative (:484)
          if (REDUCE == 0 ? (m0 > 0) : (m0 >= 0)) {
            const R depth = per_voxel ? dval : base + dval;
            project(Rm, Tv, px.ref_w, px.ref_h, depth, a.half, srcH, srcW, s);
            if (s.state == 2) {
              off = (s.fh * srcW + s.fw) * C;
              const R izz = quick_recip(s.z * s.z);
              fh = (s.h_coef * s.z - s.z_coef * s.h3d) * izz;
              fw = (s.w_coef * s.z - s.z_coef * s.w3d) * izz;
              if constexpr (FEAT)
                cnt = R(1);
              else if constexpr (AGG)  // cost_aggregate_kernels_gpu.cu.cc:388, :502
                cnt = quick_recip(static_cast<R>(REDUCE == 0 ? (int64_t)m0 * C : (int64_t)C));
              else
                cnt = quick_recip(static_cast<R>(m0));
            }
          }
        }
        rec.off[ridx + j] = off;
        rec.key[ridx + j] = off >= 0 ? ((s.fh << 16) | s.fw) : 0;
        rec.at(0, ridx + j) = s.k00;
        rec.at(1, ridx + j) = s.k01;
        rec.at(2, ridx + j) = s.k11;
        rec.at(3, ridx + j) = s.k10;
        rec.at(4, ridx + j) = s.dh;
        rec.at(5, ridx + j) = s.dw;
        rec.at(6, ridx + j) = fh;
        rec.at(7, ridx + j) = fw;
        rec.at(8, ridx + j) = cnt;
      }
      strip_sync();
      for (int nl = 0; nl < nv; ++nl) {
        const int n = n0 + nl;
        const int ridx = (nl * ppw + p) * kDB;
        const int64_t view_off = ((int64_t)px.b * N + n) * srcH * srcW * C + (ch_ok ? cl : 0);
        const S *view = a.src + view_off;
        Acc *gview = src_grad + view_off;
        if constexpr (FEAT) {  // an upstream row per view
#pragma unroll
          for (int jj = 0; jj < kDB; ++jj) {
            const int64_t i = px.pix * D + min(d0 + jj, d_hi - 1);
            cgv[jj] = Storage<S>::load(a.cost_grad + (i * N + n) * C + (ch_ok ? cl : 0));
          }
        }
        int cur = -1, have = -1;  // cell of the open run, cell whose taps are in registers
        int ckey = 0;             // the open run's cell as (row << 16) | column (cache only)
        R v00 = R(0), v01 = R(0), v11 = R(0), v10 = R(0);
        R g00 = R(0), g01 = R(0), g11 = R(0), g10 = R(0);
        if (carry) {
          cur = s_cur[n * 64 + lane];
          ckey = s_ckey[n * 64 + lane];
          g00 = s_run[(n * 4 + 0) * 64 + lane], g01 = s_run[(n * 4 + 1) * 64 + lane];
          g11 = s_run[(n * 4 + 2) * 64 + lane], g10 = s_run[(n * 4 + 3) * 64 + lane];
        }
        // The four texels of a finished run into the cache; called by all lanes of ONE pixel
        // (the tag tests are uniform among them).  The four slots of a cell are distinct; their
        // tags and values are read together, a miss writes the slot's old texel out first.
        const int img0 = (int)(((int64_t)px.b * N + n) * img_texels);  // first texel of this view's image
        auto cache_add_cell = [&]() {
          const int fh = ckey >> 16, fw = ckey & 0xffff;
          const int r0 = n * kCacheSlots + (fh & (kCacheRows - 1)) * kCacheCols;
          const int r1 = n * kCacheSlots + ((fh + 1) & (kCacheRows - 1)) * kCacheCols;
          const int c0 = fw & (kCacheCols - 1), c1 = (fw + 1) & (kCacheCols - 1);
          const int slot[4] = {r0 + c0, r0 + c1, r1 + c1, r1 + c0};
          const int t0 = img0 + fh * srcW + fw;
          const int texel[4] = {t0, t0 + 1, t0 + srcW + 1, t0 + srcW};
          const R add[4] = {g00, g01, g11, g10};
          int tag[4];
          R val[4];
#pragma unroll
          for (int k = 0; k < 4; ++k) tag[k] = s_tag[slot[k]];
#pragma unroll
          for (int k = 0; k < 4; ++k) val[k] = s_val[(size_t)slot[k] * lpp + cl];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            if (tag[k] == texel[k]) {
              val[k] += add[k];
            } else {
              if (tag[k] >= 0 && val[k] != R(0) && cl < C)
                atomic_add(src_grad + (int64_t)tag[k] * C + cl, (Acc)val[k]);
              val[k] = add[k];
              s_tag[slot[k]] = texel[k];
            }
            s_val[(size_t)slot[k] * lpp + cl] = val[k];
          }
        };
        // The lanes with `fire` (whole pixels) hand over the tap sums of their run and clear
        // them: straight to memory, or pixel by pixel into the cache (pixels of a strip hit
        // the same texels, so they must not update a slot at the same time).
        auto emit = [&](bool fire) {
          if (!cache) {
            if (fire && ch_ok) {
              Acc *q = gview + cur;
              if (g00 != R(0)) atomic_add(q, (Acc)g00);
              if (g01 != R(0)) atomic_add(q + C, (Acc)g01);
              if (g11 != R(0)) atomic_add(q + C + row_step, (Acc)g11);
              if (g10 != R(0)) atomic_add(q + row_step, (Acc)g10);
            }
          } else {
            unsigned long long m = __ballot(fire);
            while (m) {
              const int lp = (__ffsll((long long)m) - 1) >> g.lpp_shift;
              m &= ~(pix_lanes << (lp << g.lpp_shift));
              if (p == lp) cache_add_cell();
              strip_sync();
            }
          }
          g00 = g01 = g11 = g10 = R(0);  // (a lane that does not fire has no open run)
        };
#pragma unroll
        for (int jj = 0; jj < kDB; ++jj) {
          const int off = rec.off[ridx + jj];
          if (off < 0) continue;
          if (off != cur) {
            emit(cur >= 0);
            cur = off;
            ckey = rec.key[ridx + jj];
          }
          if (off != have) {
            have = off;
            const S *q = view + off;
            v00 = Storage<S>::load(q), v01 = Storage<S>::load(q + C);
            v11 = Storage<S>::load(q + C + row_step), v10 = Storage<S>::load(q + row_step);
          }
          if (!PAIR && !ch_ok) continue;
          if constexpr (REDUCE != 0)
            if (win[jj] != n) continue;  // another view won (:553)
          const R k00 = rec.at(0, ridx + jj), k01 = rec.at(1, ridx + jj), k11 = rec.at(2, ridx + jj),
                  k10 = rec.at(3, ridx + jj);
          // (CostVolumeV3 compares dot products of these samples with the forward pass's: there
          // the literal, separately rounded form)
          const R smp = PAIR ? k00 * v00 + k01 * v01 + k11 * v11 + k10 * v10
                             : mad(k10, v10, mad(k11, v11, mad(k01, v01, k00 * v00)));
          const R cg = cgv[jj];
          // CostVolumeV3 (cost_volume_kernels_gpu_v3.cu.cc:447-520, :593-640): the pair (reference
          // group gi, source group gs) this view contributed -- searched again for the mean (source
          // groups outermost, strict '<' from the smallest positive number, every dot product
          // summed in channel order from zero: the order of the forward pass, so that the same
          // pair wins), read from the mask for the MIN reduce.  All lanes of the pixel are here
          // together: the samples go through LDS.
          int gi = -1, gs = -1;
          if constexpr (PAIR) {
            s_smp[lane] = ch_ok ? smp : R(0);
            strip_sync();
            if constexpr (REDUCE == 0) {
              // lane cl takes the pairs cl, cl + LPP, ... in ascending order, then the pixel's
              // lanes compare: the larger product wins, of two equal ones the earlier pair --
              // which is what the reference's scan with '<' keeps
              const int GG = G * G;
              R best = Limits<R>::min_positive();
              int bq = -1;
              for (int q = cl; q < GG; q += lpp) {
                const int qs = q / G, qi = q - qs * G;
                R dot = R(0);
                for (int k = 0; k < sub; ++k)
                  dot += s_smp[p * lpp + qs * sub + k] * s_ref[p * lpp + qi * sub + k];
                if (best < dot) best = dot, bq = q;
              }
              for (int sh = 0; sh < g.lpp_shift; ++sh) {
                const R ov = __shfl_xor(best, 1 << sh, 64);
                const int oq = __shfl_xor(bq, 1 << sh, 64);
                if (ov > best || (ov == best && oq >= 0 && oq < bq)) best = ov, bq = oq;
              }
              // no pair above the seed: the reference indexes group -1 here (:495-496)
              if (bq < 0) continue;
              gs = bq / G, gi = bq - gs * G;
            } else {
              gi = win_gi[jj], gs = win_gs[jj];
              if (gi < 0 || gi >= G || gs < 0 || gs >= G) continue;
            }
          }
          // 1 / (views accepted): exact for 1, 2 and 4 views, else within an ulp or two of the
          // reference's division (one reciprocal per voxel in phase 1 instead of a division
          // per element)
          const R inv = rec.at(8, ridx + jj);
          R gv;
          if constexpr (FEAT) {
            gv = cg;  // feature_aggregate_kernels_gpu.cu.cc:307-311
          } else if constexpr (PAIR) {
            const R scl = REDUCE == 0 ? cg * inv : cg;  // :426, :621
            if (my_group == gi) racc = mad(scl, s_smp[p * lpp + gs * sub + my_k], racc);
            if (my_group != gs) continue;  // only the winning source group receives a gradient
            gv = scl * s_ref[p * lpp + gi * sub + my_k];
          } else if (CORR != 1) {
            const R diff = smp - ref_c;
            gv = (REDUCE == 0 || AGG) ? R(2) * diff * cg * inv : R(2) * diff * cg;  // :439, :560
            racc += -gv;
          } else {
            gv = REDUCE == 0 ? cg * inv : cg;  // v2 :461, :583
            racc = mad(gv, smp, racc);
            gv = gv * ref_c;
          }
          g00 = mad(gv, k00, g00);
          g01 = mad(gv, k01, g01);
          g11 = mad(gv, k11, g11);
          g10 = mad(gv, k10, g10);
          if (want_depth) {
            const R t1 = v11 - v10 - v01 + v00;
            const R h_grad = gv * mad(t1, rec.at(5, ridx + jj), v10 - v00);
            const R w_grad = gv * mad(t1, rec.at(4, ridx + jj), v01 - v00);
            const R dl = mad(rec.at(6, ridx + jj), h_grad, rec.at(7, ridx + jj) * w_grad);
            if (per_voxel)
              dvox[jj] += dl;
            else
              dpart += dl;
          }
        }
        if (carry) {
          s_cur[n * 64 + lane] = cur;
          s_ckey[n * 64 + lane] = ckey;
          s_run[(n * 4 + 0) * 64 + lane] = g00, s_run[(n * 4 + 1) * 64 + lane] = g01;
          s_run[(n * 4 + 2) * 64 + lane] = g11, s_run[(n * 4 + 3) * 64 + lane] = g10;
        } else {
          emit(cur >= 0);
        }
      }
    }  // group of views
    if (per_voxel && want_depth) {
#pragma unroll
      for (int jj = 0; jj < kDB; ++jj) {
        const R tot = pixel_sum(dvox[jj], g.lpp_shift);
        const int d = d0 + jj;
        // every voxel is stored, zeros on the ones the mask skips (v2 :375-378, :477)
        if (d < d_hi && px.ok && cl == 0) a.depth_grad[px.pix * D + d] = tot;
      }
    }
  }
  if (carry && ch_ok) {
    // the runs still open after the last chunk
    for (int n = 0; n < N; ++n) {
      const int cur = s_cur[n * 64 + lane];
      if (cur < 0) continue;
      Acc *q = src_grad + ((int64_t)px.b * N + n) * srcH * srcW * C + cl + cur;
      const R g00 = s_run[(n * 4 + 0) * 64 + lane], g01 = s_run[(n * 4 + 1) * 64 + lane];
      const R g11 = s_run[(n * 4 + 2) * 64 + lane], g10 = s_run[(n * 4 + 3) * 64 + lane];
      if (g00 != R(0)) atomic_add(q, (Acc)g00);
      if (g01 != R(0)) atomic_add(q + C, (Acc)g01);
      if (g11 != R(0)) atomic_add(q + C + row_step, (Acc)g11);
      if (g10 != R(0)) atomic_add(q + row_step, (Acc)g10);
    }
  }
  if (cache) {
    // everything the cache still holds
    strip_sync();
    for (int s0 = 0; s0 < N * kCacheSlots; s0 += ppw) {
      const int slot = s0 + p;
      if (slot < N * kCacheSlots && cl < C) {
        const int tag = s_tag[slot];
        if (tag >= 0) {
          const R v = s_val[(size_t)slot * lpp + cl];
          if (v != R(0)) atomic_add(src_grad + (int64_t)tag * C + cl, (Acc)v);
        }
      }
    }
  }
  if (ch_ok && !FEAT) {
    Acc *q = ref_grad + px.pix * C + cl;
    if (g.nseg == 1)
      *q = (Acc)racc;
    else
      atomic_add(q, (Acc)racc);
  }
  if (!per_voxel && want_depth) {
    const R tot = pixel_sum(dpart, g.lpp_shift);
    if (px.ok && cl == 0) {
      if (g.nseg == 1)
        a.depth_grad[px.pix] = tot;
      else
        atomic_add(a.depth_grad + px.pix, tot);
    }
  }
}



template <typename S>
StripGeom strip_geometry(const Args<S> &a) {
  StripGeom g;
  g.lpp_shift = 0;
  while ((1 << g.lpp_shift) < a.C) ++g.lpp_shift;
  const int ppw = 64 >> g.lpp_shift;
  g.tiles = (a.pixels() + ppw - 1) / ppw;
  const int lpp = 1 << g.lpp_shift;
  g.vg = lpp / kDB < 1 ? 1 : (int)(lpp / kDB < a.N ? lpp / kDB : a.N);
  // enough wavefronts to fill 256 compute units several times over, segments of whole chunks
  int nseg = 1;
  while (nseg < 16 && g.tiles * nseg < 256 * 80 && a.D / (nseg * 2) >= 2 * kDB) nseg *= 2;
  const int per = (int)((a.D + nseg - 1) / nseg);
  g.seg = (per + kDB - 1) / kDB * kDB;
  g.nseg = (int)((a.D + g.seg - 1) / g.seg);
  // carried runs: N * 64 lanes * (4 sums + tap offset + cell); given up beyond 16 KiB, or
  // where records and runs together would pass the launch limit (one channel in float64:
  // 39 KiB of records)
  using R = typename Storage<S>::Real;
  // CostVolumeV3: 64 reference values and 64 samples
  g.pair_bytes = a.corr == BEST_GROUP_PAIR ? (int)(128 * sizeof(R)) : 0;
  const size_t rec_bytes = strip_lds_bytes<R>(9, ppw * g.vg * kDB, 2) + g.pair_bytes;
  g.carry = strip_run_bytes<S>(a.N) <= 16384 && rec_bytes + strip_run_bytes<S>(a.N) <= kMaxDynamicLds;
  // Wide pixels in float64: the texel cache between the runs and memory, as long as it stays
  // small (8 KiB: four views of 32 lanes) and a texel's index over all images of the call
  // fits its 32-bit tag.  (float64 only: its atomics move twice the bytes; with 32-bit elements
  // the cache's own work costs more than it saves, 749 against 735 us at 24 channels)
  g.cache = sizeof(R) == 8 && lpp >= 16 && strip_cache_bytes<R>(a.N, lpp) <= 8192 &&
            a.B * a.N * a.srcH * a.srcW < (int64_t)1 << 31 && a.srcH < 32768 && a.srcW < 65536 &&
            rec_bytes + (g.carry ? strip_run_bytes<S>(a.N) : 0) + strip_cache_bytes<R>(a.N, lpp) <=
                kMaxDynamicLds;
  // With the cache a run that ends with its chunk costs a read-add-write in LDS, not atomics:
  // the runs are not carried then, and without their 5 KiB (two views) sixteen workgroups fit a
  // compute unit instead of thirteen -- the fourth wave per SIMD the kernel is compiled for.
  // Float64, 32 channels, two views: 995 -> 866 us for the mean's gradient, 986 -> 950 us for
  // the minimum's, 984 -> 896 us FeatureAggregate, 2810 -> 2233 us CostVolumeV3.
  if (g.cache) g.carry = 0;
  return g;
}

}  // namespace

template <typename S>
bool strip_supported(const Args<S> &a) {
  if (a.corr != SQUARED_DIFFERENCE && a.corr != GROUP_CORRELATION &&
      a.corr != SUM_SQUARED_DIFFERENCE && a.corr != WARP_ONLY)
    return false;
  if (a.C < 1 || a.C > 64 || a.N < 1 || a.D < 1 || a.pixels() < 1) return false;
  if (a.corr == GROUP_CORRELATION && (a.groups < 1 || a.C % a.groups != 0)) return false;
  if (a.srcH < 2 || a.srcW < 2) return false;                   // no sample can be accepted
  if (a.srcH * a.srcW * a.C >= (int64_t)1 << 31) return false;  // 32-bit offsets inside a view
  // per-voxel hypotheses belong to the group correlation (always) and to the squared difference
  // in 16-bit storage (by choice): the backward kernel knows this at compile time
  const bool grid = a.depth_grid != nullptr;
  if (a.corr == GROUP_CORRELATION ? !grid : grid && !(a.corr == SQUARED_DIFFERENCE && sizeof(S) == 2))
    return false;
  const StripGeom g = strip_geometry(a);
  return g.tiles * g.nseg < (int64_t)1 << 31;
}

// The gradient of CostVolumeV3 in float and double: any group width (the general kernel, one
// thread per voxel, sends every element of every tap to memory on its own).
template <typename S>
bool strip_pair_backward_supported(const Args<S> &a) {
  if constexpr (sizeof(S) == 2) {
    return false;
  } else {
    if (a.corr != BEST_GROUP_PAIR || a.depth_grid != nullptr) return false;
    if (a.C < 1 || a.C > 64 || a.N < 1 || a.D < 1 || a.pixels() < 1) return false;
    if (a.groups < 1 || a.C % a.groups != 0) return false;
    if (a.srcH < 2 || a.srcW < 2) return false;
    if (a.srcH * a.srcW * a.C >= (int64_t)1 << 31) return false;
    const StripGeom g = strip_geometry(a);
    if (a.groups > 16) return false;  // very many groups: the search of groups^2 pairs dominates
    return g.tiles * g.nseg < (int64_t)1 << 31;
  }
}

template <typename S>
hipError_t launch_strip_forward(const Args<S> &a, hipStream_t stream) {
  using R = typename Storage<S>::Real;
  const StripGeom g = strip_geometry(a);
  // CostAggregate adds one row of 64 values per depth of a chunk
  const size_t smem = strip_lds_bytes<R>(4, (64 >> g.lpp_shift) * g.vg * kDB) +
                      (a.corr == SUM_SQUARED_DIFFERENCE ? (size_t)kDB * 64 * sizeof(R) : 0);
  const dim3 grid((unsigned)(g.tiles * g.nseg)), block(64);
  if (a.corr == WARP_ONLY) {
    strip_forward_kernel<S, 4, 0><<<grid, block, smem, stream>>>(a, g);
  } else if (a.corr == SUM_SQUARED_DIFFERENCE) {
    if (a.reduce == 0)
      strip_forward_kernel<S, 2, 0><<<grid, block, smem, stream>>>(a, g);
    else
      strip_forward_kernel<S, 2, 1><<<grid, block, smem, stream>>>(a, g);
  } else if (a.corr == SQUARED_DIFFERENCE) {
    if (a.reduce == 0)
      strip_forward_kernel<S, 0, 0><<<grid, block, smem, stream>>>(a, g);
    else
      strip_forward_kernel<S, 0, 1><<<grid, block, smem, stream>>>(a, g);
  } else {
    if (a.reduce == 0)
      strip_forward_kernel<S, 1, 0><<<grid, block, smem, stream>>>(a, g);
    else
      strip_forward_kernel<S, 1, 1><<<grid, block, smem, stream>>>(a, g);
  }
  return hipGetLastError();
}

template <typename S>
hipError_t launch_strip_backward(const Args<S> &a, hipStream_t stream) {
  using R = typename Storage<S>::Real;
  const StripGeom g = strip_geometry(a);
  const int64_t n_ref = a.pixels() * a.C;
  const int64_t n_src = a.B * a.N * a.srcH * a.srcW * a.C;
  hipError_t err;
  // the scatter target starts from zero; the pixel-owned outputs only when several depth
  // segments add into them (otherwise the kernel stores every element once)
  void *src_img = sizeof(S) == 2 ? (void *)a.src_grad_acc : (void *)a.src_grad;
  void *ref_img = sizeof(S) == 2 ? (void *)a.ref_grad_acc : (void *)a.ref_grad;
  const size_t acc_size = sizeof(S) == 2 ? 4 : sizeof(S);
  ZeroRanges zero;  // one launch for all of them
  zero.add(src_img, (size_t)n_src * acc_size);
  if (g.nseg > 1) {
    if (a.corr != WARP_ONLY) zero.add(ref_img, (size_t)n_ref * acc_size);  // no reference image
    if (a.depth_grid == nullptr && a.depth_grad != nullptr)
      zero.add(a.depth_grad, (size_t)a.pixels() * sizeof(R));
  }
  if ((err = zero.launch(stream)) != hipSuccess) return err;
  const size_t smem = strip_lds_bytes<R>(9, (64 >> g.lpp_shift) * g.vg * kDB, 2) +
                      (g.carry ? strip_run_bytes<S>(a.N) : 0) +
                      (g.cache ? strip_cache_bytes<R>(a.N, 1 << g.lpp_shift) : 0) + g.pair_bytes;
  const dim3 grid((unsigned)(g.tiles * g.nseg)), block(64);
  // (float64: the four-wave form for the gradients of a mean, and for the others where the
  // texel cache is on, i.e. with wide pixels)
  constexpr bool kDouble = sizeof(S) == 8;
  const bool w4 = kDouble && g.cache;
#define CHOP_STRIP_BWD(CORR_)                                                               \
  do {                                                                                      \
    if (a.reduce == 0)                                                                      \
      strip_backward_kernel<S, CORR_, 0, kDouble><<<grid, block, smem, stream>>>(a, g);     \
    else if (w4)                                                                            \
      strip_backward_kernel<S, CORR_, 1, kDouble><<<grid, block, smem, stream>>>(a, g);     \
    else                                                                                    \
      strip_backward_kernel<S, CORR_, 1, false><<<grid, block, smem, stream>>>(a, g);       \
  } while (0)
  if (a.corr == BEST_GROUP_PAIR) {
    if constexpr (sizeof(S) != 2) CHOP_STRIP_BWD(3);
  } else if (a.corr == WARP_ONLY) {
    strip_backward_kernel<S, 4, 0, kDouble><<<grid, block, smem, stream>>>(a, g);
  } else if (a.corr == SUM_SQUARED_DIFFERENCE) {
    CHOP_STRIP_BWD(2);
  } else if (a.corr == SQUARED_DIFFERENCE) {
    CHOP_STRIP_BWD(0);
  } else {
    CHOP_STRIP_BWD(1);
  }
#undef CHOP_STRIP_BWD
  if ((err = hipGetLastError()) != hipSuccess) return err;
  if constexpr (sizeof(S) == 2) {
    if ((err = launch_narrow2<S>(a.ref_grad_acc, a.ref_grad, n_ref, a.src_grad_acc, a.src_grad, n_src,
                                 stream)) != hipSuccess)
      return err;
  }
  return hipSuccess;
}

#define CHOP_INSTANTIATE(S)                                                      \
  template bool strip_supported<S>(const Args<S> &);                             \
  template bool strip_pair_backward_supported<S>(const Args<S> &);               \
  template hipError_t launch_strip_forward<S>(const Args<S> &, hipStream_t);     \
  template hipError_t launch_strip_backward<S>(const Args<S> &, hipStream_t);
CHOP_INSTANTIATE(float)
CHOP_INSTANTIATE(double)
CHOP_INSTANTIATE(__half)
CHOP_INSTANTIATE(bf16_t)
#undef CHOP_INSTANTIATE

}  // namespace chop
