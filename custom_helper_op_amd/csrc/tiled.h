// Tiled cost-volume kernels for gfx950 (MEAN and MIN / MAX reduces, every op of the family).
//
// Work decomposition.  A workgroup is one wavefront.  It owns PPW = 64/LPP pixels of one
// image (a compact block, see tile_rows: its samples change their texel cell together more
// often than a long row's) and one contiguous segment of the D depth hypotheses; the LPP lanes
// of a pixel each own VEC consecutive channels (C = LPP*VEC), so every tap read and every
// cost-row write of a pixel is one contiguous C*sizeof(S) segment.  Depth runs innermost:
// along the walk the sample point of a view slides along an epipolar line by a fraction of
// a texel per step, so the four bilinear taps of the current texel cell stay in registers
// and are reloaded only when the cell changes.
//
// Each chunk of LPP depths is processed in two phases:
//   phase 1  lane (pixel p, j) reprojects depth d0+j of pixel p into every view (the
//            bit-exact code of warp.h), writes the valid-view count and leaves a small
//            record per (view, depth, pixel) in LDS: tap offset (or -1) and four weights
//            (backward: also the cell key and four depth-derivative weights);
//   phase 2  lane (pixel p, channel slice) walks the LPP depths, reading the records as
//            LDS broadcasts, and does the channel arithmetic with explicit fused
//            multiply-adds.
// With LPP == 1 a lane owns its whole pixel and the records stay in registers.
//
// Backward keeps, per view, a register image of the source-gradient contributions to the
// current cell.  When the cell changes the image is added into a per-view LDS
// window of ROWS x COLS texels that follows the wave's samples along the epipolar lines;
// neighbouring pixels hit the same texels, so most of the scatter is absorbed there.  A
// texel reaches memory when the window moves off it, as part of a dense run of
// global_atomic_add_f32.  ref_grad and the base-plane gradient are pixel-owned and
// accumulate in registers; they are stored once (one depth segment) or added once per
// segment.
#pragma once

#include <type_traits>

#include "internal.h"

namespace chop {
namespace tiled {

// Rows of a wave's pixel tile (PPW = 64 / LPP pixels, tile_rows x PPW / tile_rows): as square
// as the pixel count allows.  The samples of a compact tile cross texel boundaries at more
// nearly the same depths than those of a long row, so fewer wave iterations carry a cell
// change (MVSNet-stage workload, 8 pixels: 0.49 of them for 2 x 4 against 0.61 for 1 x 8;
// f16 cascade workload, 16 pixels: 0.49-0.68 per view for 4 x 4 against 0.57-0.75 for 2 x 8),
// and its footprint in the source image has fewer texels per pixel.
constexpr int tile_rows(int ppw) { return ppw >= 64 ? 8 : ppw >= 16 ? 4 : ppw >= 2 ? 2 : 1; }

struct Geometry {
  int hw;                  // H*W
  int tiles_per_image;     // ceil(hw / PPW)
  int nseg;                // depth segments
  int ngroups;             // view groups (backward only): workgroups that split the views
  int vper;                // views per group
  int seg;                 // depths per segment, multiple of LPP
  int64_t total_units;     // B * tiles_per_image * nseg * ngroups
  unsigned units_per_seg;  // B * tiles_per_image * ngroups
  int64_t units_per_xcd;   // ceil(total_units / 8)
  int xcd_shift;           // log2 of the units dealt to one XCD at a time; -1: one band per XCD
  int64_t grid;            // workgroups to launch
  int tiles_x;             // tiles per image row (a tile: tile_rows(PPW) rows of pixels)
  int sub;                 // channels per correlation group (1 for squared difference)
  float src_h_max, src_w_max;  // (float)(srcH - 1), (float)(srcW - 1): acceptance bounds
};

// ---- vector access ---------------------------------------------------------------------
template <typename S>
__device__ __forceinline__ void widen_word(uint32_t w, float *out);
template <>
__device__ __forceinline__ void widen_word<float>(uint32_t w, float *out) {
  out[0] = __uint_as_float(w);
}
template <>
__device__ __forceinline__ void widen_word<__half>(uint32_t w, float *out) {
  out[0] = __half2float(__ushort_as_half((unsigned short)(w & 0xffffu)));
  out[1] = __half2float(__ushort_as_half((unsigned short)(w >> 16)));
}
template <>
__device__ __forceinline__ void widen_word<bf16_t>(uint32_t w, float *out) {
  out[0] = __uint_as_float(w << 16);
  out[1] = __uint_as_float(w & 0xffff0000u);
}

template <typename S>
__device__ __forceinline__ uint32_t narrow_word(const float *in);
template <>
__device__ __forceinline__ uint32_t narrow_word<float>(const float *in) {
  return __float_as_uint(in[0]);
}
template <>
__device__ __forceinline__ uint32_t narrow_word<__half>(const float *in) {
  return (uint32_t)__half_as_ushort(__float2half_rn(in[0])) |
         ((uint32_t)__half_as_ushort(__float2half_rn(in[1])) << 16);
}
template <>
__device__ __forceinline__ uint32_t narrow_word<bf16_t>(const float *in) {
  return float_to_bf16_bits(in[0]) | (float_to_bf16_bits(in[1]) << 16);
}

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int BYTES>
struct Raw;
template <>
struct Raw<16> {
  using type = u32x4;
};
template <>
struct Raw<8> {
  using type = u32x2;
};
template <>
struct Raw<4> {
  using type = uint32_t;
};
template <>
struct Raw<2> {
  using type = uint16_t;
};

// Loads CNT elements of S (CNT*sizeof(S) in {2,4,8,16} bytes, naturally aligned) as floats.
// STREAM marks data that is touched once (cost rows, upstream gradients): non-temporal.
template <typename S, int CNT, bool STREAM>
__device__ __forceinline__ void load_vec(const S *p, float *out) {
  constexpr int BYTES = CNT * (int)sizeof(S);
  using RawT = typename Raw<BYTES>::type;
  constexpr int PER_WORD = 4 / (int)sizeof(S);
  const RawT *q = reinterpret_cast<const RawT *>(p);
  const RawT v = STREAM ? __builtin_nontemporal_load(q) : *q;
  if constexpr (BYTES == 2) {
    float two[2];
    widen_word<S>(v, two);
    out[0] = two[0];
  } else if constexpr (BYTES == 4) {
    widen_word<S>(v, out);
  } else {
#pragma unroll
    for (int k = 0; k < BYTES / 4; ++k) widen_word<S>(v[k], out + k * PER_WORD);
  }
}

// Output rows bypass the caches (non-temporal, STREAM) only where one store of a pixel's lanes covers
// whole 128-byte lines.  A narrower row -- 16 channels of a 16-bit type, a few correlation
// groups, the one mask word of a voxel -- shares its line with the rows of the neighbouring
// depths, which other store instructions write: streamed, each piece reaches memory on its own
// as a partial line, while L2 puts the pieces of a cached line together first (the
// valid-view counts of the MVSNet-stage forward: 134 -> 123 us).
template <typename S, int CNT, bool STREAM>
__device__ __forceinline__ void store_vec(S *p, const float *in) {
  constexpr int BYTES = CNT * (int)sizeof(S);
  using RawT = typename Raw<BYTES>::type;
  constexpr int PER_WORD = 4 / (int)sizeof(S);
  RawT *q = reinterpret_cast<RawT *>(p);
  RawT v;
  if constexpr (BYTES == 2) {
    float two[2] = {in[0], 0.f};
    v = (uint16_t)(narrow_word<S>(two) & 0xffffu);
  } else if constexpr (BYTES == 4) {
    v = narrow_word<S>(in);
  } else {
#pragma unroll
    for (int k = 0; k < BYTES / 4; ++k) v[k] = narrow_word<S>(in + k * PER_WORD);
  }
  if (STREAM)
    __builtin_nontemporal_store(v, q);
  else
    *q = v;
}

// The same load without the conversion: CNT elements as they lie in memory, in 32-bit words
// (a single 16-bit element in the low half of one word).  A wave that widens 16-bit values
// right after the load waits for memory at that point; keeping the words and widening them
// where they are used lets the wait fall behind whatever work sits in between.
template <typename S, int CNT>
constexpr int raw_words() { return (CNT * (int)sizeof(S) + 3) / 4; }
template <typename S, int CNT, bool STREAM>
__device__ __forceinline__ void load_raw(const S *p, uint32_t *out) {
  constexpr int BYTES = CNT * (int)sizeof(S);
  using RawT = typename Raw<BYTES>::type;
  const RawT *q = reinterpret_cast<const RawT *>(p);
  const RawT v = STREAM ? __builtin_nontemporal_load(q) : *q;
  if constexpr (BYTES <= 4) {
    out[0] = (uint32_t)v;
  } else {
#pragma unroll
    for (int k = 0; k < BYTES / 4; ++k) out[k] = v[k];
  }
}
template <typename S, int CNT>
__device__ __forceinline__ void widen_raw(const uint32_t *in, float *out) {
  constexpr int BYTES = CNT * (int)sizeof(S);
  constexpr int PER_WORD = 4 / (int)sizeof(S);
  if constexpr (BYTES == 2) {
    float two[2];
    widen_word<S>(in[0], two);
    out[0] = two[0];
  } else {
#pragma unroll
    for (int k = 0; k < BYTES / 4; ++k) widen_word<S>(in[k], out + k * PER_WORD);
  }
}

// (the choice is made at compile time from the row's width: a run-time test in front of every
// row store cost the MVSNet-stage forward 20 us)
constexpr bool whole_lines(int elements, int elem_bytes) { return elements * elem_bytes >= 128; }

// Orders this wave's LDS traffic: the lanes of a wavefront execute in lockstep and the
// LDS returns a wave's operations in issue order, so only the compiler has to be kept
// from moving accesses across the phase boundary.
// An LDS object at (lane-dependent byte offset) + (compile-time constant).
template <typename T>
__device__ __forceinline__ T &lds_at(unsigned char *base, unsigned lane_bytes, int const_bytes) {
  return *reinterpret_cast<T *>(base + lane_bytes + const_bytes);
}

__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Sum over each group of WIDTH consecutive lanes (WIDTH a power of two <= 16), left in every
// lane of the group.  Cross-lane moves in registers: quad permutes, then the half-row and
// row mirrors (a mirror pairs lane i with lane WIDTH-1-i; the quad steps finish the sum).
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
  return v + __int_as_float(moved);
}
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
  static_assert(WIDTH == 1 || WIDTH == 2 || WIDTH == 4 || WIDTH == 8 || WIDTH == 16, "group width");
  if constexpr (WIDTH >= 16) v = dpp_add<0x140>(v);  // row_mirror
  if constexpr (WIDTH >= 8) v = dpp_add<0x141>(v);   // row_half_mirror
  if constexpr (WIDTH >= 4) v = dpp_add<0x4E>(v);    // quad_perm 2,3,0,1
  if constexpr (WIDTH >= 2) v = dpp_add<0xB1>(v);    // quad_perm 1,0,3,2
  return v;
}

// Sums the per-channel values of each correlation group: out[g] for g < VEC/sub.
template <int VEC>
__device__ __forceinline__ void fold_groups(const float *ch, int sub, float *out) {
  if (sub == 1) {
#pragma unroll
    for (int c = 0; c < VEC; ++c) out[c] = ch[c];
  } else if (sub == 2) {
#pragma unroll
    for (int c = 0; c < VEC / 2; ++c) out[c] = ch[2 * c] + ch[2 * c + 1];
  } else if (sub == 4) {
#pragma unroll
    for (int c = 0; c < VEC / 4; ++c)
      out[c] = (ch[4 * c] + ch[4 * c + 1]) + (ch[4 * c + 2] + ch[4 * c + 3]);
  } else {  // sub == 8 == VEC
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < VEC; ++c) s += ch[c];
    out[0] = s;
  }
}

template <typename S, int VEC, int LPP>
__device__ __forceinline__ void store_groups(S *p, const float *v, int sub) {
  // p already points at this lane's first group; a pixel's row holds VEC * LPP / sub values
  constexpr int C = VEC * LPP, B = (int)sizeof(S);
  if (sub == 1) {
    store_vec<S, VEC, whole_lines(C, B)>(p, v);
  } else if (sub == 2) {
    store_vec<S, VEC / 2, whole_lines(C / 2, B)>(p, v);
  } else if (sub == 4) {
    store_vec<S, VEC / 4, whole_lines(C / 4, B)>(p, v);
  } else {
    if constexpr (VEC >= 8) store_vec<S, VEC / 8, whole_lines(C / 8, B)>(p, v);
  }
}

template <typename S, int VEC, bool STREAM>
__device__ __forceinline__ void load_groups(const S *p, float *v, int sub) {
  if (sub == 1) {
    load_vec<S, VEC, STREAM>(p, v);
  } else if (sub == 2) {
    load_vec<S, VEC / 2, STREAM>(p, v);
  } else if (sub == 4) {
    load_vec<S, VEC / 4, STREAM>(p, v);
  } else {
    if constexpr (VEC >= 8) load_vec<S, VEC / 8, STREAM>(p, v);
  }
}

// ---- shared front end of both kernels ---------------------------------------------------
template <int NV>
struct Cameras {
  float zc[NV], wc[NV], hc[NV];  // rows of R applied to (ref_w, ref_h, 1)
  float t0[NV], t1[NV], t2[NV];
};

template <int LPP>
struct Tile {
  int lane, p, cl;
  int b, pin, h, w;
  int d_lo, d_hi;
  int view0;               // first view of this workgroup's group
  bool pix_ok;
  int64_t pix;
};

template <typename S, int LPP>
__device__ __forceinline__ bool locate_tile(const Args<S> &a, const Geometry &g, Tile<LPP> &t) {
  constexpr int PPW = 64 / LPP;
  t.lane = threadIdx.x;
  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD runs of consecutive
  // tiles so that its L2 only has to hold that part of the source images.  Forward: one
  // band per XCD.  Backward: short runs, which balance the XCDs better (its tiles differ
  // more in cost).
  // (all counts fit 32 bits: the host checks total_units; 64-bit divisions would cost
  // several hundred instructions per workgroup, which runs only a few thousand)
  const unsigned bid = blockIdx.x;
  const unsigned r = bid >> 3, x = bid & 7u;
  const unsigned unit = g.xcd_shift < 0
                            ? x * (unsigned)g.units_per_xcd + r
                            : ((r >> g.xcd_shift) << (g.xcd_shift + 3)) + (x << g.xcd_shift) +
                                  (r & ((1u << g.xcd_shift) - 1u));
  if (unit >= (unsigned)g.total_units) return false;
  // the groups of one (tile, segment) are neighbours in launch order: they stream the same
  // upstream-gradient rows at about the same time, through the same L2
  unsigned tile;
  int segi;
  if (g.xcd_shift >= 0) {
    // Backward: the depth segments one after the other, all tiles of the first segment first.
    // The workgroups of a launch differ in length, and what the chip does while the last ones
    // finish is lost; the segment of the nearest hypotheses (most cell changes per depth) is
    // the longest, so it goes first and the launch ends on the shortest workgroups
    // (MVSNet-stage backward -2.5 %; the far segment first: +0.5 %).
    const unsigned sraw = unit / g.units_per_seg;
    const unsigned rem = unit - sraw * g.units_per_seg;
    segi = (int)sraw;
    tile = rem / (unsigned)g.ngroups;
    t.view0 = (int)(rem - tile * (unsigned)g.ngroups) * g.vper;
  } else {
    const unsigned per_tile = (unsigned)(g.nseg * g.ngroups);
    tile = unit / per_tile;
    const int rem = (int)(unit - tile * per_tile);
    segi = rem / g.ngroups;
    t.view0 = (rem - segi * g.ngroups) * g.vper;
  }
  t.d_lo = segi * g.seg;
  t.d_hi = min((int)a.D, t.d_lo + g.seg);
  t.b = (int)(tile / (unsigned)g.tiles_per_image);
  const int t_in = (int)(tile - (unsigned)t.b * (unsigned)g.tiles_per_image);
  t.p = t.lane / LPP;
  t.cl = t.lane % LPP;
  if constexpr (PPW == 1) {
    t.pin = t_in;
    t.pix_ok = true;
  } else {
    // A tile is tile_rows(PPW) rows of pixels: the samples of a compact tile cross texel boundaries
    // at more nearly the same depths than those of a long row, so fewer wave iterations carry
    // a cell change (0.49 against 0.62 of them on the MVSNet-stage workload).  Tiles that
    // stick out of the image have their outside pixels switched off.
    constexpr int TH = tile_rows(PPW), TW = PPW / TH;
    const int ty = t_in / g.tiles_x, tx = t_in - ty * g.tiles_x;
    const int py = t.p / TW;
    const int y = ty * TH + py, x = tx * TW + (t.p - py * TW);
    t.pix_ok = y < (int)a.H && x < (int)a.W;
    t.pin = y * (int)a.W + x;
  }
  if (!t.pix_ok) t.pin = g.hw - 1;  // clamp: loads stay in range, stores are predicated
  t.pix = (int64_t)t.b * g.hw + t.pin;
  t.h = t.pin / (int)a.W;
  t.w = t.pin - t.h * (int)a.W;
  return true;
}

template <typename S, int NV>
__device__ __forceinline__ void load_cameras(const Args<S> &a, int b, int view0, float ref_w,
                                             float ref_h, Cameras<NV> &c) {
  const int N = (int)a.N;
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    const int nn = view0 + n < N ? view0 + n : 0;
    const float *Rm = a.Rs + ((int64_t)b * N + nn) * 9;
    const float *t = a.Ts + ((int64_t)b * N + nn) * 3;
    // same association as the per-voxel expression: (R6*w + R7*h) + R8
    c.zc[n] = Rm[6] * ref_w + Rm[7] * ref_h + Rm[8];
    c.wc[n] = Rm[0] * ref_w + Rm[1] * ref_h + Rm[2];
    c.hc[n] = Rm[3] * ref_w + Rm[4] * ref_h + Rm[5];
    c.t0[n] = t[0], c.t1[n] = t[1], c.t2[n] = t[2];
  }
}

// One reprojection with hoisted row products; bit-identical to warp.h's project().
struct Hit {
  int off;     // element offset of tap (fh,fw) inside the view's image, or -1
  int key;     // (fh << 16) | fw
  float k00, k01, k11, k10;
  float dh, dw;
  float z, w3d, h3d;
};

template <int NV>
__device__ __forceinline__ void reproject(const Cameras<NV> &c, int n, float depth, float half,
                                          float src_h_max, float src_w_max, int srcW, int C,
                                          Hit &r) {
  r.off = -1;
  r.key = 0;
  r.k00 = r.k01 = r.k11 = r.k10 = 0.f;
  r.z = c.zc[n] * depth + c.t2[n];
  if (r.z <= 0.f) return;
  r.w3d = c.wc[n] * depth + c.t0[n];
  float sw = r.w3d / r.z;
  r.h3d = c.hc[n] * depth + c.t1[n];
  float sh = r.h3d / r.z;
  sw = sw - half;
  sh = sh - half;
  if (sh > 0.f && sw > 0.f && sh < src_h_max && sw < src_w_max) {
    const int fh = static_cast<int>(sh), fw = static_cast<int>(sw);
    r.dh = sh - static_cast<float>(fh);
    r.dw = sw - static_cast<float>(fw);
    r.k11 = r.dh * r.dw;
    r.k10 = r.dh * (1.f - r.dw);
    r.k00 = (1.f - r.dh) * (1.f - r.dw);
    r.k01 = (1.f - r.dh) * r.dw;
    r.off = (fh * srcW + fw) * C;
    r.key = (fh << 16) | fw;
  }
}

template <typename S>
__device__ __forceinline__ float voxel_depth(const Args<S> &a, int64_t pix, int b, int d,
                                             float base) {
  return a.depth_grid ? a.depth_grid[pix * a.D + d] : base + a.offsets[(int64_t)b * a.D + d];
}

// =========================================================================================
// Forward
// =========================================================================================
// Stores CNT (1, 2 or 4) consecutive int32 values; STREAM as for the cost rows.
template <int CNT, bool STREAM>
__device__ __forceinline__ void store_ints(int32_t *p, const int *v) {
  constexpr bool stream = STREAM;
  if constexpr (CNT == 4) {
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    i32x4 w = {v[0], v[1], v[2], v[3]};
    if (stream) __builtin_nontemporal_store(w, reinterpret_cast<i32x4 *>(p));
    else *reinterpret_cast<i32x4 *>(p) = w;
  } else if constexpr (CNT == 2) {
    typedef int i32x2 __attribute__((ext_vector_type(2)));
    i32x2 w = {v[0], v[1]};
    if (stream) __builtin_nontemporal_store(w, reinterpret_cast<i32x2 *>(p));
    else *reinterpret_cast<i32x2 *>(p) = w;
  } else {
    if (stream) __builtin_nontemporal_store(v[0], p);
    else *p = v[0];
  }
}

// ---- CostVolumeV3: the largest correlation of any source group with any reference group ------
// A value of another lane of the same pixel, in registers.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ int dpp_move(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}
// One butterfly step of "largest value, earliest pair on a tie" (both partners end equal).
template <int CTRL>
__device__ __forceinline__ void better_pair(float &best, int &code) {
  const float ob = dpp_move<CTRL>(best);
  const int oc = dpp_move<CTRL>(code);
  const bool take = ob > best || (ob == best && oc < code);
  best = take ? ob : best;
  code = take ? oc : code;
}
constexpr int kNoPair = 0x7fffffff;  // pair code: source group * 16 + reference group

// The best (source group, reference group) pair of one accepted sample of one pixel, found
// by the pixel's LPP lanes exactly as the reference's loop finds it
// (cost_volume_kernels_gpu_v3.cu.cc:113-130): lane cl holds the sample of channels
// 4cl..4cl+3, i.e. part (cl % (SUB/4)) of group cl / (SUB/4); every dot product is one
// sequential chain over the group's channels, each product and sum rounded separately (for 8
// channels the even lane's partial sum continues in the odd lane); source group outermost,
// strict "<" from the smallest positive float, so the earliest pair keeps a tie.
// `ref_row`: the pixel's reference channels in LDS.  Every lane of the pixel returns the same
// best value (the seed when no pair exceeds it) and pair code (kNoPair then).
template <int VEC, int LPP, int SUB>
__device__ __forceinline__ void v3_best_pair(const float (&smp)[VEC], const float *ref_row, int cl,
                                             float &best, int &code) {
  static_assert(VEC == 4 && (SUB == 4 || SUB == 8), "a group is one lane or two");
  constexpr int C = VEC * LPP, G = C / SUB, LPG = SUB / 4;
  typedef float f4 __attribute__((ext_vector_type(4)));
  const int group = cl / LPG, koff = (cl % LPG) * 4;
  best = __FLT_MIN__;
  code = kNoPair;
#pragma unroll
  for (int gi = 0; gi < G; ++gi) {
    const f4 r = *reinterpret_cast<const f4 *>(ref_row + gi * SUB + koff);
    const float p0 = smp[0] * r[0], p1 = smp[1] * r[1], p2 = smp[2] * r[2], p3 = smp[3] * r[3];
    float dot = ((p0 + p1) + p2) + p3;  // (0 + p0 differs from p0 in the sign of zero only)
    if constexpr (LPG == 2) {
      const float head = dpp_move<0xA0>(dot);  // quad_perm 0,0,2,2: the even lane's four terms
      dot = (((head + p0) + p1) + p2) + p3;    // complete in the odd lane
    }
    if (best < dot) {
      best = dot;
      code = group * 16 + gi;
    }
  }
  if constexpr (LPG == 2) {
    if ((cl & 1) == 0) best = __FLT_MIN__, code = kNoPair;
  }
  if constexpr (LPP >= 2) better_pair<0xB1>(best, code);    // quad_perm 1,0,3,2
  if constexpr (LPP >= 4) better_pair<0x4E>(best, code);    // quad_perm 2,3,0,1
  if constexpr (LPP >= 8) better_pair<0x141>(best, code);   // row_half_mirror
  if constexpr (LPP >= 16) better_pair<0x140>(best, code);  // row_mirror
}

// The gradient of one accepted sample flows through one pair: the view's best pair, found
// again as in the forward (REDUCE 0, :469-491), or the recorded winner `pair` (REDUCE 1).
// Out: gsrc = d(loss)/d(sample) of this lane's channels (zero outside the winning source
// group); racc += the reference gradient of this lane's channels (zero outside the winning
// reference group, :494-512).  `rows` = two LDS arrays of 64*VEC floats: the pixel rows of
// the reference image (written once by the caller) and of this sample.
template <int VEC, int LPP, int SUB, int REDUCE>
__device__ __forceinline__ void v3_pair_gradients(const float4 wt, const float (&tap)[4][VEC],
                                                  float cg, int pair, float *rows, int p, int cl,
                                                  float (&racc)[VEC], float (&gsrc)[VEC]) {
  constexpr int C = VEC * LPP, LPG = SUB / 4;
  typedef float f4 __attribute__((ext_vector_type(4)));
  float *ref_row = rows + p * C, *smp_row = rows + 64 * VEC + p * C;
  const int group = cl / LPG, koff = (cl % LPG) * 4;
  float smp[VEC];
#pragma unroll
  for (int c = 0; c < 4; ++c)
    smp[c] = wt.x * tap[0][c] + wt.y * tap[1][c] + wt.z * tap[2][c] + wt.w * tap[3][c];
  *reinterpret_cast<f4 *>(smp_row + cl * 4) = f4{smp[0], smp[1], smp[2], smp[3]};
  int code = pair;
  if constexpr (REDUCE == 0) {
    float best;
    v3_best_pair<VEC, LPP, SUB>(smp, ref_row, cl, best, code);
  }
  const bool any = code != kNoPair;
  const int gi_w = code & 15, gs_w = code >> 4;
#pragma unroll
  for (int c = 0; c < 4; ++c) gsrc[c] = 0.f;
  if (any && group == gs_w) {
    const f4 r = *reinterpret_cast<const f4 *>(ref_row + gi_w * SUB + koff);
#pragma unroll
    for (int c = 0; c < 4; ++c) gsrc[c] = cg * r[c];
  }
  wave_sync();  // the sample row is complete
  if (any && group == gi_w) {
    const f4 m = *reinterpret_cast<const f4 *>(smp_row + gs_w * SUB + koff);
#pragma unroll
    for (int c = 0; c < 4; ++c) racc[c] = __builtin_fmaf(cg, m[c], racc[c]);
  }
}

// The first workgroups of a forward launch read one word of every 128-byte line of the source
// and reference images, 128 lines per workgroup, so that the images stream into the memory-side
// cache at the start of the launch.  Without it a launch that finds them in no cache spends its
// first tens of microseconds on tap gathers that each wait for HBM (MVSNet-stage forward after
// the caches have been overwritten: 152 -> 127 us; no difference when the images are cached).
// Only for images of up to 16 MB together: larger ones do not stay in the caches anyway, and
// touching them costs the launch their size in extra reads (f16 cascade workload, 29 MB:
// forward 95 -> 107 us with it).
// The values are not used; keep_alive() at the end of the kernel keeps the loads in the code.
struct Touched {
  unsigned a, b;
};
template <typename S>
__device__ __forceinline__ Touched touch_images(const Args<S> &a) {
  Touched w{0u, 0u};
  const size_t src_bytes = (size_t)a.B * a.N * a.srcH * a.srcW * a.C * sizeof(S);
  const size_t ref_bytes = a.ref != nullptr ? (size_t)a.B * a.H * a.W * a.C * sizeof(S) : 0;
  const size_t o0 = ((size_t)blockIdx.x * 128 + threadIdx.x) * 128, o1 = o0 + 64 * 128;
  if (src_bytes + ref_bytes <= ((size_t)16 << 20) && o0 < src_bytes + ref_bytes) {  // (uniform)
    const char *sb = reinterpret_cast<const char *>(a.src), *rb = reinterpret_cast<const char *>(a.ref);
    if (o0 + 4 <= src_bytes)
      w.a = *reinterpret_cast<const unsigned *>(sb + o0);
    else if (o0 >= src_bytes && o0 - src_bytes + 4 <= ref_bytes)
      w.a = *reinterpret_cast<const unsigned *>(rb + (o0 - src_bytes));
    if (o1 + 4 <= src_bytes)
      w.b = *reinterpret_cast<const unsigned *>(sb + o1);
    else if (o1 >= src_bytes && o1 - src_bytes + 4 <= ref_bytes)
      w.b = *reinterpret_cast<const unsigned *>(rb + (o1 - src_bytes));
  }
  return w;
}
__device__ __forceinline__ void keep_alive(const Touched &w) {
  asm volatile("" ::"v"(w.a), "v"(w.b));  // no instruction: the two registers count as read here
}

template <int NV>
constexpr int forward_lds_words(int lpp) {
  return lpp > 1 ? NV * 64 * 5 : 0;
}
// The minimum of the summed squared difference also stages one chunk of squares per view:
// a row of C (+4 padding, so that the eight readers of a pixel hit different banks) floats
// per (pixel, depth).
constexpr int forward_squares_words(int lpp) { return lpp > 1 ? 64 * (4 * lpp + 4) : 0; }

// REDUCE: 0 mean over the accepted views (mask = their number), 1 per-channel minimum of
// the squared difference / per-group maximum of the correlation with the winning view as
// mask (-1: none).  The winner must be the reference's, so that reduce uses the literal
// operand order with every operation rounded separately instead of the fused chains.
// Minimum waves per SIMD the register allocator has to leave room for (mean of the squared
// difference or of the group correlation only: the MIN / MAX reduces keep winner indices per
// depth and channel and would spill).  Five and six views: left alone the compiler takes ~140
// registers (three waves); held to 128 it needs no scratch, and the fourth wave hides the tap
// gathers of wide-baseline views (stress workload forward 5.17 -> 4.45 ms).  Three and four
// views at four lanes per pixel: 102 -> 87 registers without scratch, five waves instead of
// four (f16 cascade workload forward 122 -> 113 us cold); the other widths would spill.
constexpr int forward_min_waves(int lpp, int nv, int corr, int reduce) {
  if (corr > 1 || reduce != 0) return 1;
  return nv >= 5 ? 4 : (nv >= 3 && lpp == 4) ? 5 : 1;
}

template <typename S, int VEC, int LPP, int NV, int CORR, int REDUCE = 0>
// At most five waves per SIMD: with six (the two-view instantiation needs only 80 VGPRs)
// the waves of a CU evict each other's taps from L1 and the kernel is 6 % slower.  The lower
// bound: see forward_min_waves.
__global__ __launch_bounds__(64)
__attribute__((amdgpu_waves_per_eu(forward_min_waves(LPP, NV, CORR, REDUCE), 5))) void forward_kernel(
    const Args<S> a, const Geometry g) {
  constexpr int PPW = 64 / LPP;
  extern __shared__ __align__(16) unsigned char smem[];
  Tile<LPP> t;
  // (one or two views only: the instantiations for more views are held to a register budget
  // that two more live registers break -- f16 cascade forward 95 -> 107 us with them)
  Touched touched{0u, 0u};
  if constexpr (NV <= 2) touched = touch_images(a);
  if (!locate_tile<S, LPP>(a, g, t)) {
    if constexpr (NV <= 2) keep_alive(touched);
    return;
  }
  const int C = (int)a.C, D = (int)a.D, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW;
  const float half = a.half;
  // LDS records: wts[NV][LPP][PPW] then off[NV][LPP][PPW], addressed as (lane-dependent
  // byte offset) + (compile-time constant) so that the constant lands in the instruction's
  // offset field instead of costing a register per unrolled depth
  constexpr int kWts = 0, kOff = NV * 64 * 16;
  const unsigned p4 = (unsigned)t.p * 4u;                 // reader: pixel p
  const unsigned q4 = (unsigned)(t.cl * PPW + t.p) * 4u;  // writer: lane (p, j)

  Cameras<NV> cam;
  load_cameras<S, NV>(a, t.b, t.view0, static_cast<float>(t.w) + half,
                      static_cast<float>(t.h) + half, cam);
  const float base = a.depth_grid ? 0.f : a.base_plane[t.pix];
  float ref[VEC];
  if constexpr (CORR != 4) {
    load_vec<S, VEC, false>(a.ref + t.pix * C + t.cl * VEC, ref);
    if constexpr (CORR == 3) {
      // CostVolumeV3: every lane of a pixel reads all of the pixel's reference groups
      static_assert(CORR != 3 || (LPP > 1 && VEC == 4), "CostVolumeV3: wide pixels");
      float *s_ref = reinterpret_cast<float *>(smem + NV * 64 * 20);  // behind the records
#pragma unroll
      for (int c = 0; c < VEC; ++c) s_ref[t.p * (VEC * LPP) + t.cl * VEC + c] = ref[c];
      wave_sync();
    }
  } else {
#pragma unroll
    for (int c = 0; c < VEC; ++c) ref[c] = 0.f;  // the warp-only op has no reference image
  }
  const S *view[NV];
#pragma unroll
  for (int n = 0; n < NV; ++n)
    view[n] = a.src + ((int64_t)t.b * N + (n < N ? n : 0)) * srcH * srcW * C + t.cl * VEC;
  const int row_step = srcW * C;

  float tap[NV][4][VEC];
  int cur[NV];
#pragma unroll
  for (int n = 0; n < NV; ++n) cur[n] = -1;

  // CORR: 0 squared difference per channel, 1 group correlation, 2 squared difference
  // summed over all channels (one value per voxel), 4 the samples themselves, one row per
  // (voxel, view), and a 0/1 mask per (voxel, view)
  // (feature_aggregate_kernels_gpu.cu.cc:33-121)
  // 3: CostVolumeV3, per view the largest correlation of any (source group, reference group)
  // pair; MEAN averages the views' maxima, MIN keeps the largest with (view, reference group,
  // source group) as its mask (cost_volume_kernels_gpu_v3.cu.cc:52-146, :148-262)
  const int OC = CORR == 1 ? a.groups : (CORR == 2 || CORR == 3) ? 1 : C;
  const int gv = VEC / g.sub;  // output values per lane
  // the cost rows of the per-channel ops (and the sample rows of the warp-only op) stream past
  // the caches where they cover whole lines
  constexpr bool kNtRows = whole_lines(VEC * LPP, (int)sizeof(S));
  const int d_lo = t.d_lo, d_hi = t.d_hi;
  // the cost-map layers' default fill folded into the store: where no view was accepted the
  // scalar is written instead of the cost (custom_layers.py:52-57, :78-83)
  const bool fill = a.default_cost != nullptr;
  const float dflt = fill ? *a.default_cost : 0.f;
  // this pixel's output rows (the 64-bit product once per wave, not once per depth)
  S *const out_pix = a.cost + t.pix * D * OC;
  int32_t *const mask_pix = a.mask + t.pix * D * OC;
  for (int d0 = d_lo; d0 < d_hi; d0 += LPP) {
    // ---- phase 1: reprojection by lane (p, j = cl) --------------------------------------
    int r_off[NV];
    float4 r_wts[NV];
    unsigned vmask = 0u;  // views accepted for lane (p, j)'s own voxel
    {
      const int d = d0 + t.cl;
      const bool d_ok = d < d_hi;
      const float depth = d_ok ? voxel_depth(a, t.pix, t.b, d, base) : 1.f;
      int cnt = 0;
#pragma unroll
      for (int n = 0; n < NV; ++n) {
        Hit hit;
        hit.off = -1;
        hit.k00 = hit.k01 = hit.k11 = hit.k10 = 0.f;
        if (n < N && d_ok) reproject<NV>(cam, n, depth, half, g.src_h_max, g.src_w_max, srcW, C, hit);
        cnt += hit.off >= 0;
        if constexpr (CORR == 2 && REDUCE == 1) vmask |= (hit.off >= 0 ? 1u : 0u) << n;
        if constexpr (CORR == 4) {
          if (n < N && d_ok && t.pix_ok)
            a.mask[(t.pix * D + d) * N + n] = hit.off >= 0 ? 1 : 0;
        }
        if constexpr (LPP > 1) {
          lds_at<int>(smem, q4, kOff + (n * LPP * PPW) * 4) = hit.off;
          lds_at<float4>(smem, q4 * 4u, kWts + (n * LPP * PPW) * 16) =
              make_float4(hit.k00, hit.k01, hit.k11, hit.k10);
        } else {
          r_off[n] = hit.off;
          r_wts[n] = make_float4(hit.k00, hit.k01, hit.k11, hit.k10);
        }
      }
      if constexpr (REDUCE == 0 && CORR != 4)
        if (d_ok && t.pix_ok) a.mask[t.pix * D + d] = cnt;
    }
    if constexpr (LPP > 1) wave_sync();
    if constexpr (CORR == 2 && REDUCE == 1) {
      // Minimum over the views of the squared difference summed over ALL channels
      // (cost_aggregate_kernels_gpu.cu.cc:128-229).  The mask names the winning view, so the
      // sum has to be the reference's: channel 0 first, every product and sum rounded
      // separately.  View by view, the channel lanes leave the chunk's squares in LDS and the
      // lane that owns voxel (p, d0 + cl) adds its row up in channel order.
      constexpr int kSq = NV * 64 * 20;             // behind the records
      constexpr int ROWB = (VEC * LPP + 4) * 4;     // bytes per (pixel, depth) row
      float best = 3.402823466e+38f;                // numeric_limits<T>::max(), :170
      int win = -1;
#pragma unroll
      for (int n = 0; n < NV; ++n) {
        float own = 0.f;  // LPP == 1: this lane holds the whole pixel
#pragma unroll
        for (int jj = 0; jj < LPP; ++jj) {
          if (d0 + jj >= d_hi) {
            if constexpr (LPP >= 16) continue; else break;
          }
          int off;
          float4 wt;
          if constexpr (LPP > 1) {
            off = lds_at<int>(smem, p4, kOff + ((n * LPP + jj) * PPW) * 4);
            wt = lds_at<float4>(smem, p4 * 4u, kWts + ((n * LPP + jj) * PPW) * 16);
          } else {
            off = r_off[n];
            wt = r_wts[n];
          }
          float sq[VEC];
#pragma unroll
          for (int c = 0; c < VEC; ++c) sq[c] = 0.f;
          if (off >= 0) {
            if (off != cur[n]) {
              cur[n] = off;
              const S *q = view[n] + off;
              load_vec<S, VEC, false>(q, tap[n][0]);
              load_vec<S, VEC, false>(q + C, tap[n][1]);
              load_vec<S, VEC, false>(q + row_step + C, tap[n][2]);
              load_vec<S, VEC, false>(q + row_step, tap[n][3]);
            }
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
              const float smp = wt.x * tap[n][0][c] + wt.y * tap[n][1][c] + wt.z * tap[n][2][c] +
                                wt.w * tap[n][3][c];
              const float diff = smp - ref[c];
              sq[c] = diff * diff;
            }
          }
          if constexpr (LPP > 1) {
            lds_at<float4>(smem, (unsigned)(t.p * LPP * ROWB + t.cl * VEC * 4), kSq + jj * ROWB) =
                make_float4(sq[0], sq[1], sq[2], sq[3]);
          } else {
            own = 0.f;
#pragma unroll
            for (int c = 0; c < VEC; ++c) own += sq[c];
          }
        }
        if constexpr (LPP > 1) {
          wave_sync();
          if ((vmask >> n) & 1u) {
            float tot = 0.f;
#pragma unroll
            for (int k = 0; k < LPP; ++k) {
              const float4 v = lds_at<float4>(
                  smem, (unsigned)((t.p * LPP + t.cl) * ROWB), kSq + k * VEC * 4);
              tot += v.x;
              tot += v.y;
              tot += v.z;
              tot += v.w;
            }
            if (best > tot) best = tot, win = n;  // strict: the earliest view keeps a tie (:217)
          }
          wave_sync();
        } else {
          if (((vmask >> n) & 1u) && best > own) best = own, win = n;
        }
      }
      const int d = d0 + t.cl;
      if (d < d_hi && t.pix_ok) {
        const float out = win >= 0 ? best / static_cast<float>(C) : dflt;  // :222-227
        reinterpret_cast<float *>(a.cost)[t.pix * D + d] = out;
        a.mask[t.pix * D + d] = win;
      }
      continue;
    }
    if constexpr ((CORR == 0 || CORR == 1) && (NV >= 5 || (NV >= 3 && LPP == 4))) {
      // ---- phase 2, one view at a time (many views) ---------------------------------------
      // With every view's four taps live at once the kernel needs ~25 registers per view
      // (171 for six views: two waves per SIMD).  Here a block of up to eight depths keeps
      // its accumulators and the views take turns with one set of taps, so the register count
      // hardly depends on the number of views.  Every accumulator still receives the views in
      // order 0..N-1 with the same operations, so the results are those of the
      // depth-by-depth loop.  (Measurements decide where this form is used: for three or four
      // views the depth-by-depth loop needs fewer registers at 32+ channels, and with one or
      // two lanes per pixel its taps, which survive from chunk to chunk, matter more.)
      constexpr int DB = LPP < 8 ? LPP : 8;
#pragma unroll
      for (int j0 = 0; j0 < LPP; j0 += DB) {
      float acc[DB][VEC];
      int arg[REDUCE == 1 ? DB : 1][VEC];
      int kcnt[DB];
#pragma unroll
      for (int jj = 0; jj < DB; ++jj) {
        kcnt[jj] = 0;
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
          acc[jj][c] = REDUCE == 0 ? 0.f : CORR == 0 ? 3.402823466e+38f : 1.175494351e-38f;
          if constexpr (REDUCE == 1) arg[jj][c] = -1;
        }
      }
#pragma unroll
      for (int n = 0; n < NV; ++n) {
        int cur1 = -1;
        float tp[4][VEC];
#pragma unroll
        for (int jj = 0; jj < DB; ++jj) {
          if (d0 + j0 + jj >= d_hi) continue;
          int off;  // -1 also for a view beyond N (phase 1 leaves those records empty)
          if constexpr (LPP > 1)
            off = lds_at<int>(smem, p4, kOff + ((n * LPP + j0 + jj) * PPW) * 4);
          else
            off = r_off[n];
          if (off < 0) continue;
          float4 wt;
          if constexpr (LPP > 1)
            wt = lds_at<float4>(smem, p4 * 4u, kWts + ((n * LPP + j0 + jj) * PPW) * 16);
          else
            wt = r_wts[n];
          if (off != cur1) {
            cur1 = off;
            const S *q = view[n] + off;
            load_vec<S, VEC, false>(q, tp[0]);
            load_vec<S, VEC, false>(q + C, tp[1]);
            load_vec<S, VEC, false>(q + row_step + C, tp[2]);
            load_vec<S, VEC, false>(q + row_step, tp[3]);
          }
          ++kcnt[jj];
          if constexpr (REDUCE == 1) {
            float val[VEC];
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
              const float smp = wt.x * tp[0][c] + wt.y * tp[1][c] + wt.z * tp[2][c] + wt.w * tp[3][c];
              if (CORR == 0) {
                const float diff = smp - ref[c];
                val[c] = diff * diff;
              } else {
                val[c] = smp * ref[c];
              }
            }
            if (CORR == 0) {
#pragma unroll
              for (int c = 0; c < VEC; ++c)
                if (acc[jj][c] > val[c]) acc[jj][c] = val[c], arg[jj][c] = n;
            } else {
#pragma unroll
              for (int gi = 0; gi < VEC; ++gi) {
                if (gi * g.sub < VEC) {
                  float corr = 0.f;
#pragma unroll
                  for (int c = 0; c < VEC; ++c)
                    if (c >= gi * g.sub && c < (gi + 1) * g.sub) corr += val[c];
                  if (acc[jj][gi] < corr) acc[jj][gi] = corr, arg[jj][gi] = n;
                }
              }
            }
          } else {
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
              if (CORR != 1) {
                float diff = __builtin_fmaf(wt.x, tp[0][c], -ref[c]);
                diff = __builtin_fmaf(wt.y, tp[1][c], diff);
                diff = __builtin_fmaf(wt.z, tp[2][c], diff);
                diff = __builtin_fmaf(wt.w, tp[3][c], diff);
                acc[jj][c] = __builtin_fmaf(diff, diff, acc[jj][c]);
              } else {
                float smp = wt.x * tp[0][c];
                smp = __builtin_fmaf(wt.y, tp[1][c], smp);
                smp = __builtin_fmaf(wt.z, tp[2][c], smp);
                smp = __builtin_fmaf(wt.w, tp[3][c], smp);
                acc[jj][c] = __builtin_fmaf(smp, ref[c], acc[jj][c]);
              }
            }
          }
        }
      }
#pragma unroll
      for (int jj = 0; jj < DB; ++jj) {
        const int d = d0 + j0 + jj;
        if (d >= d_hi || !t.pix_ok) continue;
        S *out = out_pix + d * OC;  // d * OC is uniform: one add per lane
        if constexpr (REDUCE == 1) {
          int32_t *mout = mask_pix + d * OC;
          if (fill) {
#pragma unroll
            for (int c = 0; c < VEC; ++c)
              if (arg[jj][c] < 0) acc[jj][c] = dflt;
          }
          if (CORR == 0) {
            store_vec<S, VEC, kNtRows>(out + t.cl * VEC, acc[jj]);
            store_ints<VEC, whole_lines(VEC * LPP, 4)>(mout + t.cl * VEC, arg[jj]);
          } else {
            store_groups<S, VEC, LPP>(out + t.cl * gv, acc[jj], g.sub);
            if (g.sub == 1) store_ints<VEC, whole_lines(VEC * LPP, 4)>(mout + t.cl * gv, arg[jj]);
            else if (g.sub == 2) store_ints<VEC / 2, whole_lines(VEC * LPP / 2, 4)>(mout + t.cl * gv, arg[jj]);
            else store_ints<VEC / 4, whole_lines(VEC * LPP / 4, 4)>(mout + t.cl * gv, arg[jj]);
          }
        } else {
          if (kcnt[jj] > 1) {
            const float inv = __builtin_amdgcn_rcpf(static_cast<float>(kcnt[jj]));
#pragma unroll
            for (int c = 0; c < VEC; ++c) acc[jj][c] *= inv;
          }
          if (CORR == 0) {
            if (fill && kcnt[jj] == 0) {
#pragma unroll
              for (int c = 0; c < VEC; ++c) acc[jj][c] = dflt;
            }
            store_vec<S, VEC, kNtRows>(out + t.cl * VEC, acc[jj]);
          } else {
            float grp[VEC];
            fold_groups<VEC>(acc[jj], g.sub, grp);
            if (fill && kcnt[jj] == 0) {
#pragma unroll
              for (int c = 0; c < VEC; ++c) grp[c] = dflt;
            }
            store_groups<S, VEC, LPP>(out + t.cl * gv, grp, g.sub);
          }
        }
      }
      }  // block of depths
      if constexpr (LPP > 1) wave_sync();
      continue;
    }
    float agg_out = 0.f;
    int v3_out[3] = {-1, -1, -1};
    // ---- phase 2: channel arithmetic by lane (p, channel slice) ---------------------------
#pragma unroll
    for (int jj = 0; jj < LPP; ++jj) {
      const int d = d0 + jj;
      if (d >= d_hi) {
        // (a `break` gives the widest tile a run-time trip count, which keeps the compiler
        // from unrolling it and sends its register arrays to scratch memory)
        if constexpr (LPP >= 16) continue; else break;
      }
      float acc[VEC];
      int arg[VEC];  // REDUCE == 1: winning view per channel (or per group)
#pragma unroll
      for (int c = 0; c < VEC; ++c) {
        // numeric_limits::max() / ::min() seeds, cost_volume_kernels_gpu.cu.cc:174-177 and
        // cost_volume_kernels_gpu_v2.cu.cc:179
        acc[c] = REDUCE == 0 ? 0.f : CORR == 0 ? 3.402823466e+38f : 1.175494351e-38f;
        arg[c] = -1;
      }
      int k = 0;
      float v3_acc = REDUCE == 0 ? 0.f : 1.175494351e-38f;  // :76, :193
      int v3_view = -1, v3_code = 0;
#pragma unroll
      for (int n = 0; n < NV; ++n) {
        int off;
        float4 wt;
        if constexpr (LPP > 1) {
          off = lds_at<int>(smem, p4, kOff + ((n * LPP + jj) * PPW) * 4);
          wt = lds_at<float4>(smem, p4 * 4u, kWts + ((n * LPP + jj) * PPW) * 16);
        } else {
          off = r_off[n];
          wt = r_wts[n];
        }
        if constexpr (CORR == 3) {
          if (off >= 0) {
            if (off != cur[n]) {
              cur[n] = off;
              const S *q = view[n] + off;
              load_vec<S, VEC, false>(q, tap[n][0]);
              load_vec<S, VEC, false>(q + C, tap[n][1]);
              load_vec<S, VEC, false>(q + row_step + C, tap[n][2]);
              load_vec<S, VEC, false>(q + row_step, tap[n][3]);
            }
            float smp[VEC];
#pragma unroll
            for (int c = 0; c < VEC; ++c)
              smp[c] = wt.x * tap[n][0][c] + wt.y * tap[n][1][c] + wt.z * tap[n][2][c] +
                       wt.w * tap[n][3][c];
            const float *ref_row =
                reinterpret_cast<const float *>(smem + NV * 64 * 20) + t.p * (VEC * LPP);
            float best;
            int code;
            if (g.sub == 8)
              v3_best_pair<VEC, LPP, 8>(smp, ref_row, t.cl, best, code);
            else
              v3_best_pair<VEC, LPP, 4>(smp, ref_row, t.cl, best, code);
            if constexpr (REDUCE == 0) {
              v3_acc += best;  // the seed when no pair exceeds it (:113-131)
            } else if (v3_acc < best) {
              // one running maximum over views and pairs (:231-250)
              v3_acc = best, v3_view = n, v3_code = code;
            }
            ++k;
          }
          continue;
        }
        if constexpr (CORR == 4) {
          // the sample in the reference's operand order (bit-identical to the plain
          // evaluation), zeros for a view that is not accepted
          float smp[VEC];
#pragma unroll
          for (int c = 0; c < VEC; ++c) smp[c] = 0.f;
          if (off >= 0) {
            if (off != cur[n]) {
              cur[n] = off;
              const S *q = view[n] + off;
              load_vec<S, VEC, false>(q, tap[n][0]);
              load_vec<S, VEC, false>(q + C, tap[n][1]);
              load_vec<S, VEC, false>(q + row_step + C, tap[n][2]);
              load_vec<S, VEC, false>(q + row_step, tap[n][3]);
            }
#pragma unroll
            for (int c = 0; c < VEC; ++c)
              smp[c] = wt.x * tap[n][0][c] + wt.y * tap[n][1][c] + wt.z * tap[n][2][c] +
                       wt.w * tap[n][3][c];
          }
          if (n < N && t.pix_ok)
            store_vec<S, VEC, kNtRows>(a.cost + ((t.pix * D + d) * N + n) * C + t.cl * VEC, smp);
          continue;
        }
        if (off >= 0) {
          if (off != cur[n]) {
            cur[n] = off;
            const S *q = view[n] + off;
            load_vec<S, VEC, false>(q, tap[n][0]);
            load_vec<S, VEC, false>(q + C, tap[n][1]);
            load_vec<S, VEC, false>(q + row_step + C, tap[n][2]);
            load_vec<S, VEC, false>(q + row_step, tap[n][3]);
          }
          if constexpr (REDUCE == 1) {
            float val[VEC];
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
              const float smp = wt.x * tap[n][0][c] + wt.y * tap[n][1][c] + wt.z * tap[n][2][c] +
                                wt.w * tap[n][3][c];
              if (CORR == 0) {
                const float diff = smp - ref[c];
                val[c] = diff * diff;
              } else {
                val[c] = smp * ref[c];
              }
            }
            if (CORR == 0) {
#pragma unroll
              for (int c = 0; c < VEC; ++c)
                if (acc[c] > val[c]) acc[c] = val[c], arg[c] = n;
            } else {
              // groups of sub consecutive channels, summed in channel order from zero
#pragma unroll
              for (int gi = 0; gi < VEC; ++gi) {
                if (gi * g.sub < VEC) {
                  float corr = 0.f;
#pragma unroll
                  for (int c = 0; c < VEC; ++c)
                    if (c >= gi * g.sub && c < (gi + 1) * g.sub) corr += val[c];
                  if (acc[gi] < corr) acc[gi] = corr, arg[gi] = n;
                }
              }
            }
            ++k;
            continue;
          }
#pragma unroll
          for (int c = 0; c < VEC; ++c) {
            if (CORR != 1) {
              // sample - ref as one chain of fused multiply-adds
              float diff = __builtin_fmaf(wt.x, tap[n][0][c], -ref[c]);
              diff = __builtin_fmaf(wt.y, tap[n][1][c], diff);
              diff = __builtin_fmaf(wt.z, tap[n][2][c], diff);
              diff = __builtin_fmaf(wt.w, tap[n][3][c], diff);
              acc[c] = __builtin_fmaf(diff, diff, acc[c]);
            } else {
              float smp = wt.x * tap[n][0][c];
              smp = __builtin_fmaf(wt.y, tap[n][1][c], smp);
              smp = __builtin_fmaf(wt.z, tap[n][2][c], smp);
              smp = __builtin_fmaf(wt.w, tap[n][3][c], smp);
              acc[c] = __builtin_fmaf(smp, ref[c], acc[c]);
            }
          }
          ++k;
        }
      }
      if constexpr (CORR == 4) continue;  // every view's row is already stored
      if constexpr (CORR == 3) {
        // the lane whose slice index equals the depth's place in the chunk keeps the voxel
        if (t.cl == jj) {
          if constexpr (REDUCE == 0) {
            agg_out = k > 0 ? v3_acc / static_cast<float>(k) : 0.f;  // :136-141
          } else {
            agg_out = v3_view >= 0 ? v3_acc : 0.f;  // :253-257
            v3_out[0] = v3_view;
            v3_out[1] = v3_view >= 0 ? (v3_code & 15) : -1;
            v3_out[2] = v3_view >= 0 ? (v3_code >> 4) : -1;
          }
        }
        continue;
      }
      if constexpr (REDUCE == 1) {
        if (fill) {
#pragma unroll
          for (int c = 0; c < VEC; ++c)
            if (arg[c] < 0) acc[c] = dflt;
        }
        if (t.pix_ok) {
          S *out = out_pix + d * OC;  // d * OC is uniform: one add per lane
          int32_t *mout = mask_pix + d * OC;
          if (CORR == 0) {
            store_vec<S, VEC, kNtRows>(out + t.cl * VEC, acc);
            store_ints<VEC, whole_lines(VEC * LPP, 4)>(mout + t.cl * VEC, arg);
          } else {
            store_groups<S, VEC, LPP>(out + t.cl * gv, acc, g.sub);
            if (g.sub == 1) store_ints<VEC, whole_lines(VEC * LPP, 4)>(mout + t.cl * gv, arg);
            else if (g.sub == 2) store_ints<VEC / 2, whole_lines(VEC * LPP / 2, 4)>(mout + t.cl * gv, arg);
            else store_ints<VEC / 4, whole_lines(VEC * LPP / 4, 4)>(mout + t.cl * gv, arg);
          }
        }
        continue;
      }
      if constexpr (CORR == 2) {
        // one value per voxel: the pixel's lanes add up their channels; the lane whose
        // slice index equals the depth's place in the chunk keeps the result, so that the
        // chunk is stored as LPP consecutive floats per pixel
        float tot = group_sum<LPP>((acc[0] + acc[1]) + (acc[2] + acc[3]));
        tot = k > 0 ? tot / static_cast<float>(k * C) : dflt;
        if constexpr (LPP > 1) {
          if (t.cl == jj) agg_out = tot;
        } else {
          if (t.pix_ok) reinterpret_cast<float *>(a.cost)[t.pix * D + d] = tot;
        }
        continue;
      }
      if (k > 1) {
        const float inv = __builtin_amdgcn_rcpf(static_cast<float>(k));
#pragma unroll
        for (int c = 0; c < VEC; ++c) acc[c] *= inv;
      }
      if (t.pix_ok) {
        S *out = out_pix + d * OC;  // d * OC is uniform: one add per lane
        if (CORR == 0) {
          if (fill && k == 0) {
#pragma unroll
            for (int c = 0; c < VEC; ++c) acc[c] = dflt;
          }
          store_vec<S, VEC, kNtRows>(out + t.cl * VEC, acc);
        } else {
          float grp[VEC];
          fold_groups<VEC>(acc, g.sub, grp);
          if (fill && k == 0) {
#pragma unroll
            for (int c = 0; c < VEC; ++c) grp[c] = dflt;
          }
          store_groups<S, VEC, LPP>(out + t.cl * gv, grp, g.sub);
        }
      }
    }
    if constexpr ((CORR == 2 || CORR == 3) && LPP > 1) {
      if (t.pix_ok && d0 + t.cl < d_hi)
        reinterpret_cast<float *>(a.cost)[t.pix * D + d0 + t.cl] = agg_out;
    }
    if constexpr (CORR == 3 && REDUCE == 1) {
      if (t.pix_ok && d0 + t.cl < d_hi) {
        int32_t *m = a.mask + (t.pix * D + d0 + t.cl) * 3;
        m[0] = v3_out[0], m[1] = v3_out[1], m[2] = v3_out[2];
      }
    }
    if constexpr (LPP > 1) wave_sync();
  }
  if constexpr (NV <= 2) keep_alive(touched);
}

// =========================================================================================
// Backward
// =========================================================================================
// Per-view scatter window: a ring buffer of ROWS x COLS texels (C fp32 sums each) addressed
// by the low bits of the texel coordinates.  `oy, ox` is the window origin: the window
// holds exactly the texels [oy, oy+ROWS) x [ox, ox+COLS).  Because the slot of a texel
// depends only on its coordinates, the four slots of a cell are computed once, by the lane
// that reprojects the voxel, and travel with the record.
template <int VEC, int LPP, bool SIX = false>
struct Window {
  static constexpr int PPW = 64 / LPP;
  // twice the tile's height by twice its width, at least eight each way: room for the
  // samples' drift in either direction (8 x 8 against 4 x 16 for the 2 x 4 pixels of 32
  // channels: 357 -> 338 us on the MVSNet-stage workload)
  static constexpr int TH = tile_rows(PPW), TW = PPW / TH;
  // SIX (eight lanes per pixel, 32 channels, 2 x 4 pixels, kernels held to four waves per
  // SIMD: see backward_waves): six rows instead of eight.  With a 6 KB window the workgroup's
  // LDS is 10 KB, so that sixteen workgroups fit a CU; four rows measured 2 % slower than eight
  // at equal occupancy, six sit between.  The ring index of a row is then a remainder, not a
  // mask.
  static constexpr int ROWS = SIX ? 6 : (2 * TH > 8 ? 2 * TH : 8);
  static constexpr int COLS = 2 * TW > 8 ? 2 * TW : 8;
  static constexpr int SLOTS = ROWS * COLS;
  static constexpr bool kPow2Rows = (ROWS & (ROWS - 1)) == 0;
  // ring row of image row `fh` (not negative)
  static __device__ __forceinline__ int ring_row(unsigned fh) {
    return kPow2Rows ? (int)(fh & (unsigned)(ROWS - 1)) : (int)(fh % (unsigned)ROWS);
  }
  // image row of ring row `ry` for a window whose first row is `oy` (any sign)
  static __device__ __forceinline__ int image_row(int ry, int oy) {
    if constexpr (kPow2Rows) {
      return oy + ((ry - oy) & (ROWS - 1));
    } else {
      int m = (ry - oy) % ROWS;
      return oy + (m < 0 ? m + ROWS : m);
    }
  }
  static constexpr int C = VEC * LPP;
  static constexpr int STRIDE = C;      // one slot = C consecutive words: 16-byte lane accesses
  static constexpr int kNone = 0x3fffffff;
  static constexpr bool kPacked = SLOTS <= 256;  // four slot numbers fit one word
  static constexpr int kInside = (int)0x80000000u;  // flag in the key word: cell lies in the window

  // slots of the taps 00, 01, 11, 10 of cell `key`, one byte each
  static __device__ __forceinline__ unsigned pack_slots(int key) {
    const int fh = (key >> 16) & 0x7fff, fw = key & 0xffff;
    const int ry0 = ring_row((unsigned)fh) * COLS, ry1 = ring_row((unsigned)fh + 1u) * COLS;
    const int rx0 = fw & (COLS - 1), rx1 = (fw + 1) & (COLS - 1);
    return (unsigned)(ry0 + rx0) | ((unsigned)(ry0 + rx1) << 8) | ((unsigned)(ry1 + rx1) << 16) |
           ((unsigned)(ry1 + rx0) << 24);
  }
  // whole cell inside the window at origin (oy, ox)?
  static __device__ __forceinline__ bool inside(int key, int oy, int ox) {
    const int fh = (key >> 16) & 0x7fff, fw = key & 0xffff;
    return (unsigned)(fh - oy) < (unsigned)(ROWS - 1) && (unsigned)(fw - ox) < (unsigned)(COLS - 1);
  }
};

// Pixels of up to this many lanes update the scatter window in claimed tap-by-tap rounds
// (see window_add), which needs one claim word per window slot.
constexpr int kClaimLanes = 8;

// LDS words of the backward kernel: the records of one chunk
//   float4 wts, dwt [NV*64] | int off [NV*64] | int2 cell {slots, key|inside} [NV*64] |
//   float scale [64] | float dst [64]
// then the list of texels leaving a window, then the windows.  With one view per workgroup
// the list shares the record space: a window only moves before the chunk's records are
// written.
template <int VEC, int LPP, int NV, bool SIX = false>
constexpr int backward_record_words() {
  using WN = Window<VEC, LPP, SIX>;
  const int rec = LPP > 1 ? NV * 64 * 11 + 128 : 0;
  const int list = WN::SLOTS * 2;
  const int w = NV == 1 ? (rec > list ? rec : list) : rec + list;
  return (w + 3) / 4 * 4;
}
template <int VEC, int LPP, int NV, bool SIX = false>
constexpr int backward_lds_words() {
  using WN = Window<VEC, LPP, SIX>;
  // records (or list), windows, one cell (4 texels x C) staged on its way to memory, and for
  // narrow pixels one claim word per window slot
  return backward_record_words<VEC, LPP, NV, SIX>() + NV * WN::SLOTS * WN::STRIDE + 4 * WN::C +
         (LPP <= kClaimLanes ? WN::SLOTS : 0);
}

// Minimum over the 64 lanes, in registers: four DPP steps reduce each row of 16 lanes,
// four lane reads combine the rows.
__device__ __forceinline__ int wave_min(int v) {
  v = min(v, __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xf, 0xf, false));   // quad_perm 1,0,3,2
  v = min(v, __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xf, 0xf, false));   // quad_perm 2,3,0,1
  v = min(v, __builtin_amdgcn_update_dpp(v, v, 0x141, 0xf, 0xf, false));  // row_half_mirror
  v = min(v, __builtin_amdgcn_update_dpp(v, v, 0x140, 0xf, 0xf, false));  // row_mirror
  return min(min(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
             min(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

// Moves the window of one view to origin (ny, nx): every texel that falls outside the new
// window is written out with dense global atomics (C consecutive floats per texel, 64/C
// texels per instruction) and its slot is cleared.  Uniform control flow.
template <int VEC, int LPP, bool SIX = false>
__device__ __forceinline__ void window_move(int &oy, int &ox, int ny, int nx, float *data,
                                            int *list, float *gview, int srcW, int lane) {
  using WN = Window<VEC, LPP, SIX>;
  if (oy != WN::kNone) {
    wave_sync();  // the adds of the chunk before are complete and visible
    int count = 0;
    for (int sb = 0; sb < WN::SLOTS; sb += 64) {
      const int s = sb + lane;  // (a window of 48 slots: the last lanes have none)
      const int ry = s / WN::COLS, rx = s % WN::COLS;
      const int y = WN::image_row(ry, oy), x = ox + ((rx - ox) & (WN::COLS - 1));
      const bool leaving = s < WN::SLOTS && !((unsigned)(y - ny) < (unsigned)WN::ROWS &&
                                              (unsigned)(x - nx) < (unsigned)WN::COLS);
      const unsigned long long m = __ballot(leaving);
      if (leaving) {
        const int rank = count + (int)__builtin_amdgcn_mbcnt_hi(
            (unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u));  // leaving lanes below me
        list[2 * rank] = s;
        list[2 * rank + 1] = y * srcW + x;
      }
      count += __popcll(m);
    }
    if (count > 0) {
      wave_sync();
      constexpr int EPI = 64 / WN::C;  // texels per instruction
      constexpr int UN = 4;            // instructions per round: their LDS reads go out together
      const int sub_e = lane / WN::C, j = lane - sub_e * WN::C;
      const int2 *pairs = reinterpret_cast<const int2 *>(list);
      for (int e0 = 0; e0 < count; e0 += UN * EPI) {
        int2 le[UN];
        float v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          const int e = e0 + u * EPI + sub_e;
          le[u] = pairs[e < count ? e : 0];
          if (e >= count) le[u].x = -1;
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) v[u] = le[u].x >= 0 ? data[le[u].x * WN::STRIDE + j] : 0.f;
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          if (v[u] != 0.f) {
            data[le[u].x * WN::STRIDE + j] = 0.f;
            atomic_add(gview + (int64_t)le[u].y * WN::C + j, v[u]);
          }
        }
      }
      wave_sync();
    }
  }
  oy = ny;
  ox = nx;
}

// Bitwise OR over the 64 lanes, in registers (as wave_min).
__device__ __forceinline__ unsigned wave_or(unsigned v) {
  v |= (unsigned)__builtin_amdgcn_update_dpp((int)v, (int)v, 0xB1, 0xf, 0xf, false);
  v |= (unsigned)__builtin_amdgcn_update_dpp((int)v, (int)v, 0x4E, 0xf, 0xf, false);
  v |= (unsigned)__builtin_amdgcn_update_dpp((int)v, (int)v, 0x141, 0xf, 0xf, false);
  v |= (unsigned)__builtin_amdgcn_update_dpp((int)v, (int)v, 0x140, 0xf, 0xf, false);
  return (unsigned)__builtin_amdgcn_readlane((int)v, 0) | (unsigned)__builtin_amdgcn_readlane((int)v, 16) |
         (unsigned)__builtin_amdgcn_readlane((int)v, 32) | (unsigned)__builtin_amdgcn_readlane((int)v, 48);
}

// Writes out everything a window holds, when its view is done: row by row of the ring
// buffer, and only the rows some accepted cell of this view ever mapped to (`rows`: bit r
// set when a cell used ring row r; a short sweep over few hypotheses touches three or four
// of the eight, and the untouched ones need neither their LDS reads nor their address
// arithmetic).  All LDS reads of a row are issued together, then its atomics.
template <int VEC, int LPP, bool SIX = false>
__device__ __forceinline__ void window_flush_all(int oy, int ox, const float *data, float *gview,
                                                 int srcW, int lane, unsigned rows) {
  using WN = Window<VEC, LPP, SIX>;
  if (oy == WN::kNone) return;
  wave_sync();  // the last adds are complete and visible
  constexpr int C = WN::C;
  constexpr int PER_ROW = WN::COLS * C / 64;  // instructions of 64 consecutive floats per row
  static_assert(WN::COLS * C % 64 == 0, "whole instructions per window row");
  if (__popc(rows) > WN::ROWS * 5 / 8) {
    // (nearly) every row in use, as after a long sweep: the whole window in batches of 32
    // instructions whose LDS reads go out together, so that the wave waits for the LDS once
    // per batch instead of once per row (315 against 325 us on the MVSNet-stage workload)
    constexpr int NI = WN::SLOTS * C / 64;
    constexpr int BATCH = NI < 32 ? NI : 32;
    static_assert(NI % BATCH == 0, "whole batches");
#pragma unroll 1
    for (int i0 = 0; i0 < NI; i0 += BATCH) {
      float v[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; ++u) v[u] = data[(i0 + u) * 64 + lane];
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        const int e = (i0 + u) * 64 + lane;  // float index inside the window
        const int sl = e / C, ch = e - sl * C;
        const int ry = sl / WN::COLS, rx = sl - ry * WN::COLS;
        const int y = WN::image_row(ry, oy), x = ox + ((rx - ox) & (WN::COLS - 1));
        if (v[u] != 0.f) atomic_add(gview + ((int64_t)(y * srcW + x) * C + ch), v[u]);
      }
    }
    return;
  }
#pragma unroll 1
  for (int ry = 0; ry < WN::ROWS; ++ry) {
    if (!((rows >> ry) & 1u)) continue;  // uniform
    const int y = WN::image_row(ry, oy);
    float v[PER_ROW];
#pragma unroll
    for (int u = 0; u < PER_ROW; ++u) v[u] = data[(ry * PER_ROW + u) * 64 + lane];
#pragma unroll
    for (int u = 0; u < PER_ROW; ++u) {
      const int e = u * 64 + lane;  // float index inside the row
      const int rx = e / C, ch = e - rx * C;
      const int x = ox + ((rx - ox) & (WN::COLS - 1));
      // (a slot that was never added to holds zero: texels outside the image never are)
      if (v[u] != 0.f) atomic_add(gview + ((int64_t)(y * srcW + x) * C + ch), v[u]);
    }
  }
}

// Adds the four tap images of a finished run into the window (a cell that sticks out of the
// window never gets here: flush_cells_to_memory takes it).  Called from divergent code by all
// LPP lanes of every pixel whose run just ended.  Float LDS atomics cost about three cycles
// per lane, so the window sums are updated with plain 16-byte read-add-write.  Cells of
// different pixels overlap (a texel is tap 01 of one cell and tap 00 of its neighbour).
// Up to kClaimLanes lanes per pixel (8 to 64 pixels per wave, from two to a dozen firing at
// once): all firing pixels add tap 00, then all tap 01, ... — two pixels then collide only
// if they are on the SAME cell, and those are told apart by a claim: every pending pixel
// writes its number into the claim word of its first texel's slot and the one that reads its
// own number back goes ahead; the others try again (`tags`: one word per slot).  A pixel that
// fires alone skips all that.  Against one pixel per round this takes the headline backward
// from 429 to 400 us; against LDS atomics it halved the time of the 8-channel workloads.
// 16 lanes per pixel (four pixels per wave): the pixels that fire in the same instruction
// take turns, one pixel per round with its four taps in flight together.
template <int VEC, int LPP, bool LEAN = false, bool SIX = false>
__device__ __forceinline__ void window_add(unsigned slots, int key, float (&v)[4][VEC],
                                           float *data, int *tags, int lane, int cl) {
  using WN = Window<VEC, LPP, SIX>;
  typedef float vecf __attribute__((ext_vector_type(VEC)));
  if (key < 0) {
    // the whole cell lies inside the window (the usual case)
    if constexpr (!WN::kPacked) slots = 0;
    int slot[4];
    if constexpr (WN::kPacked) {
      slot[0] = slots & 255u, slot[1] = (slots >> 8) & 255u, slot[2] = (slots >> 16) & 255u,
      slot[3] = slots >> 24;
    } else {
      const int fh = (key >> 16) & 0x7fff, fw = key & 0xffff;
      const int ry0 = WN::ring_row((unsigned)fh) * WN::COLS, ry1 = WN::ring_row((unsigned)fh + 1u) * WN::COLS;
      const int rx0 = fw & (WN::COLS - 1), rx1 = (fw + 1) & (WN::COLS - 1);
      slot[0] = ry0 + rx0, slot[1] = ry0 + rx1, slot[2] = ry1 + rx1, slot[3] = ry1 + rx0;
    }
    float *base = data + cl * VEC;
    if constexpr (LPP > kClaimLanes) {
      unsigned long long firing = __ballot(true);
      while (firing) {
        const int lead = __ffsll((long long)firing) - 1;
        firing &= ~(((1ull << LPP) - 1ull) << lead);  // retire this pixel's lanes
        if (lane - cl == lead) {
          vecf old[4];
#pragma unroll
          for (int k = 0; k < 4; ++k)
            old[k] = *reinterpret_cast<vecf *>(base + slot[k] * WN::STRIDE);
#pragma unroll
          for (int k = 0; k < 4; ++k) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) old[k][i] += v[k][i];
            *reinterpret_cast<vecf *>(base + slot[k] * WN::STRIDE) = old[k];
          }
        }
        if (firing) wave_sync();
      }
    } else {
      const int me = lane - cl;  // the same in all lanes of a pixel
      bool pending = true;
      if (__popcll(__ballot(true)) == LPP) {
        // one pixel alone (four of ten events on the headline workload): nothing to
        // collide with, its four taps go in flight together -- or, in a kernel held to a
        // register budget, one after the other (twelve registers less at the kernel's peak)
        if constexpr (LEAN) {
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            vecf old = *reinterpret_cast<vecf *>(base + slot[k] * WN::STRIDE);
#pragma unroll
            for (int i = 0; i < VEC; ++i) old[i] += v[k][i];
            *reinterpret_cast<vecf *>(base + slot[k] * WN::STRIDE) = old;
          }
        } else {
          vecf old[4];
#pragma unroll
          for (int k = 0; k < 4; ++k)
            old[k] = *reinterpret_cast<vecf *>(base + slot[k] * WN::STRIDE);
#pragma unroll
          for (int k = 0; k < 4; ++k) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) old[k][i] += v[k][i];
            *reinterpret_cast<vecf *>(base + slot[k] * WN::STRIDE) = old[k];
          }
        }
        pending = false;
      }
      while (pending) {
        if (pending) tags[slot[0]] = me;
        wave_sync();
        const bool go = pending && tags[slot[0]] == me;
        if (go) {
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            vecf *d = reinterpret_cast<vecf *>(base + slot[k] * WN::STRIDE);
            vecf old = *d;
#pragma unroll
            for (int i = 0; i < VEC; ++i) old[i] += v[k][i];
            *d = old;
            // (the next tap may be the texel another pixel has just updated: the LDS keeps a
            // wave's operations in order, the compiler is held to it here)
            wave_sync();
          }
        }
        pending = pending && !go;
        if (__ballot(pending) == 0ull) break;
      }
      wave_sync();
    }
  }
  // (a cell that sticks out of the window never gets here: flush_cells_to_memory took it)
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[k][i] = 0.f;
}

// Cells that stick out of the window (samples of consecutive depths jumping far apart, as
// they do close to the cameras) go to memory directly.  Uniform control flow: `m` has the
// lane bits of every pixel with such a cell (`mine` for the caller's own lanes).  One pixel
// at a time, its lanes lay the four tap images out in LDS as two rows of two adjacent texels
// and the whole wave adds each row as a dense run of 2*C consecutive floats.  Added lane by
// lane from the registers, each 16-byte chunk of a texel would carry one float per
// instruction, and the atomics cost per chunk, not per float.
template <int VEC, int LPP>
__device__ __forceinline__ void flush_cells_to_memory(unsigned long long m, bool mine, int key,
                                                      float (&v)[4][VEC], float *stage,
                                                      float *gview, int srcW, int lane, int cl) {
  constexpr int C = VEC * LPP;
  typedef float vecf __attribute__((ext_vector_type(VEC)));
  while (m) {
    const int lead = __ffsll((long long)m) - 1;
    m &= ~(((1ull << LPP) - 1ull) << lead);
    const int k2 = __builtin_amdgcn_readlane(key, lead);  // the same in all lanes of the pixel
    if (lane - cl == lead) {
      // taps 00, 01 (row fh), then 10, 11 (row fh + 1); v is ordered 00, 01, 11, 10
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        vecf w;
#pragma unroll
        for (int i = 0; i < VEC; ++i) w[i] = v[k][i];
        *reinterpret_cast<vecf *>(stage + (k == 2 ? 3 : k == 3 ? 2 : k) * C + cl * VEC) = w;
      }
    }
    wave_sync();
    const int fh = k2 >> 16, fw = k2 & 0xffff;
    float *row0 = gview + (int64_t)(fh * srcW + fw) * C;
    float *row1 = row0 + (int64_t)srcW * C;
#pragma unroll
    for (int f0 = 0; f0 < 2 * C; f0 += 64) {
      const int f = f0 + lane;
      if (f < 2 * C) {
        const float a0 = stage[f], a1 = stage[2 * C + f];
        if (a0 != 0.f) atomic_add(row0 + f, a0);
        if (a1 != 0.f) atomic_add(row1 + f, a1);
      }
    }
    wave_sync();
  }
  if (mine) {
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[k][i] = 0.f;
  }
}

// Waves per SIMD the register budget is held to.  The kernel is latency-bound (its time
// falls in proportion to the resident waves), so one view per workgroup at three waves
// beats two views at two, and four waves beat three wherever registers and LDS allow them.
// Eight lanes per pixel (32 channels), gradient of the mean squared difference: 161 registers
// left alone.  Held to 128 it spills 80 bytes in the depth loop, so the kernel is slimmed
// first (lean_backward): four upstream rows staged at a time instead of eight (16 registers),
// the records of a depth read where the depth starts instead of one depth ahead (10), the
// four window taps of a pixel that fires alone added one after the other (12) -- 127 registers,
// no scratch.  Those three cost 5 % at three waves per SIMD; with the 10 KB of LDS of the
// six-row window the fourth wave gains 11 % (MVSNet-stage backward 301 -> 277 us).
// Likewise the gradients of CostAggregate (both reduces: 137 -> 117 registers) and of
// FeatureAggregate (149 -> 119).  Not the MIN / MAX gradients of the per-channel ops (their mask
// rows keep them above 140) and not CostVolumeV3 (its two extra LDS rows per pixel are 2 KB).
// Four lanes per pixel (16 channels), gradients of a mean: 130 registers left alone, 121 lean
// (held to 128 without the slimming they spilled three to five); the window of the 4 x 4 pixel
// tile is 4 KB.  Two lanes per pixel (8 channels): 119-125 lean, and 122-128 where the views of
// a tile take turns in the workgroup (VLOOP) -- once the compiler is kept from carrying two
// dozen lane-only values through the view loop (see the barrier at the head of that loop;
// with them the kernels spilled 44-68 bytes around the depth loop and four waves were slower
// than three).  Up to 32 bytes of scratch remain in two of those instantiations, outside the
// depth loop: bf16 group-correlation backward 479 -> 462 us cold, 447 -> 417 us warm.
constexpr bool lean_backward(int nv, int lpp, int corr, int reduce, bool wide = false) {
  return nv == 1 && !wide && ((lpp == 8 && ((corr == 0 && reduce == 0) || corr == 2 || corr == 4)) ||
                     (lpp == 4 && corr <= 1 && reduce == 0) ||
                     (lpp == 2 && corr <= 1 && reduce == 0));
}
constexpr int backward_waves(int nv, int lpp, int corr = 0, int reduce = 1, bool wide = false) {
  return lean_backward(nv, lpp, corr, reduce, wide) ? 4
         : nv == 1 && lpp <= 8                       ? 3
         : nv <= 2                                   ? 2
                                                     : 1;
}

// REDUCE: 0 gradient of the mean (mask = number of accepted views), 1 gradient of the
// per-channel minimum / per-group maximum (mask = winning view per channel or group; a
// voxel is skipped when its first entry is negative, cost_volume_kernels_gpu.cu.cc:483-486)
// and of the summed-squared-difference minimum (mask = the voxel's winning view).
// DG: false when the caller does not want the depth gradient (a NULL output): the four
// depth-derivative weights per record and the 20 instructions per wave-iteration that use
// them drop out.
// PV: the depth hypotheses come from a per-voxel depth_grid (and the depth gradient is per
// voxel); a compile-time flag, because the kernel without the unused variant's code is
// measurably faster than one that tests a.depth_grid at run time.
// VLOOP: the workgroup's view group holds several views, which take turns (g.vper of them).
// A compile-time flag: the loop around the kernel's body costs the wide instantiations
// registers they do not have (the 32-channel kernel spills with it).
// WIDE: the kernel as it is without the slimming of lean_backward: three waves per SIMD and, for
// 32 channels, the 8 x 8 window.  For sweeps whose samples of consecutive hypotheses land many
// texels apart (wide baselines, hypotheses close to the cameras) the two rows more are worth
// more than the fourth wave: fewer cells stick out of the window and go to memory on their
// own, and such launches are bound by those atomics, not by latency (six source views with
// 15-degree rotations and depths from 0.5: 18.9 ms against 20.6 ms slimmed).  The launcher
// decides (tiled_launch.inc).
template <typename S, int VEC, int LPP, int NV, int CORR, int REDUCE = 0, bool DG = true,
          bool PV = (CORR == 1), bool VLOOP = false, bool WIDE = false>
__global__ __launch_bounds__(64, backward_waves(NV, LPP, CORR, REDUCE, WIDE)) void backward_kernel(const Args<S> a,
                                                                          const Geometry g) {
  constexpr bool kLean = lean_backward(NV, LPP, CORR, REDUCE, WIDE);
  constexpr bool kSix = kLean && LPP == 8;
  using WN = Window<VEC, LPP, kSix>;
  constexpr int PPW = 64 / LPP;
  constexpr bool kWide = sizeof(S) == 2;  // gradients accumulate in fp32 images
  extern __shared__ __align__(16) unsigned char smem[];
  Tile<LPP> t;
  if (!locate_tile<S, LPP>(a, g, t)) return;
  const int C = (int)a.C, D = (int)a.D, N = (int)a.N, srcH = (int)a.srcH, srcW = (int)a.srcW;
  const float half = a.half;
  constexpr bool per_voxel_depth = PV;
  // byte offsets of the record arrays; a record is addressed as (lane-dependent byte offset)
  // + (compile-time constant), so that the constant lands in the instruction's offset field
  constexpr int kWts = 0, kDwt = kWts + NV * 64 * 16, kCell = kDwt + NV * 64 * 16,
                kOff = kCell + NV * 64 * 8, kScl = kOff + NV * 64 * 4, kDst = kScl + 64 * 4;
  const unsigned p4 = (unsigned)t.p * 4u;                      // reader: pixel p
  const unsigned q4 = (unsigned)(t.cl * PPW + t.p) * 4u;       // writer: lane (p, j)
  int *s_list = NV == 1 ? reinterpret_cast<int *>(smem)
                        : reinterpret_cast<int *>(smem) + (LPP > 1 ? NV * 64 * 11 + 128 : 0);
  float *s_data = reinterpret_cast<float *>(smem) + backward_record_words<VEC, LPP, NV, kSix>();
  float *s_stage = s_data + NV * WN::SLOTS * WN::STRIDE;
  int *s_tags = reinterpret_cast<int *>(s_stage + 4 * WN::C);  // narrow pixels: claim words
  static_assert(LPP > kClaimLanes || NV == 1, "one set of claim words: one view per workgroup");
  // CORR 3 only: reference rows, sample rows
  float *s_v3 = s_stage + 4 * WN::C + (LPP <= kClaimLanes ? WN::SLOTS : 0);
  static_assert(CORR != 3 || (NV == 1 && LPP > 1 && VEC == 4), "CostVolumeV3: one view, wide pixels");
  const float base = per_voxel_depth ? 0.f : a.base_plane[t.pix];
  float ref[VEC];
  if constexpr (CORR != 4) {
    load_vec<S, VEC, false>(a.ref + t.pix * C + t.cl * VEC, ref);
    if constexpr (CORR == 3) {
#pragma unroll
      for (int c = 0; c < VEC; ++c) s_v3[t.p * (VEC * LPP) + t.cl * VEC + c] = ref[c];
    }
  } else {
    static_assert(CORR != 4 || NV == 1, "the warp-only gradient runs one view per workgroup");
#pragma unroll
    for (int c = 0; c < VEC; ++c) ref[c] = 0.f;
  }
  const int64_t view_elems = (int64_t)srcH * srcW * C;
  float *src_grad_img = kWide ? a.src_grad_acc : reinterpret_cast<float *>(a.src_grad);
  const int row_step = srcW * C;
  const unsigned lane_ch = (unsigned)(t.cl * VEC);
  float racc[VEC];
#pragma unroll
  for (int c = 0; c < VEC; ++c) racc[c] = 0.f;
  float dacc = 0.f;  // base-plane gradient partial of this lane

  // CORR: 0 squared difference per channel, 1 group correlation, 2 squared difference
  // summed over all channels (one upstream gradient per voxel), 4 the warp alone: one
  // upstream-gradient row and one 0/1 mask entry per (voxel, view)
  // (feature_aggregate_kernels_gpu.cu.cc:219-326)
  // 3: CostVolumeV3, one upstream gradient per voxel that flows through the best group pair
  constexpr bool kVoxelGrad = CORR == 2 || CORR == 3;
  const int OC = CORR == 1 ? a.groups : kVoxelGrad ? 1 : C;
  const int gv = VEC / g.sub;
  const int d_lo = t.d_lo, d_hi = t.d_hi;
  // upstream-gradient rows fetched ahead; the MIN reduce stages the mask rows beside them
  constexpr int PFMAX = (REDUCE || kLean) ? 4 : 8;
  constexpr int PF = LPP < PFMAX ? LPP : PFMAX;
  constexpr bool kMaskRows = REDUCE == 1 && !kVoxelGrad;
  // mask entries per voxel: the MIN reduce of CostVolumeV3 records (view, reference group,
  // source group)
  const int mask_w = kMaskRows ? OC : (CORR == 3 && REDUCE == 1) ? 3 : 1;
  // element steps from one depth to the next in the upstream gradient and in the mask
  const int cg_step = CORR == 4 ? N * C : OC;
  const int cnt_step = CORR == 4 ? N : mask_w;
  const float *dv_src = per_voxel_depth ? a.depth_grid + t.pix * D : a.offsets + (int64_t)t.b * D;
  // The views of this workgroup's group take turns (NV at a time; NV = 1 in every launch):
  // each gets the scatter window to itself and leaves it empty.  What belongs to the pixel
  // (reference gradient, depth gradients, the upstream rows in the caches) is shared, so a
  // group of all N views needs no atomics for the pixel-owned outputs.
  const int first_view = t.view0;
  const int group_views = VLOOP ? min(g.vper > NV ? g.vper : NV, N - first_view) : NV;
  for (int vi = 0; vi < group_views; vi += NV) {
  t.view0 = first_view + vi;
  if constexpr (VLOOP) {
    // The lane index as a value the compiler cannot see through: without this it computes
    // everything that depends only on the lane (slot and row arithmetic of the window moves
    // and flushes) once in front of the view loop and keeps it in registers through all
    // views -- two dozen registers the depth loop needs.
    asm volatile("" : "+v"(t.lane), "+v"(t.cl), "+v"(t.p), "+v"(t.pix), "+v"(t.h), "+v"(t.w));
  }
  for (int k = t.lane * 4; k < NV * WN::SLOTS * WN::STRIDE; k += 256)
    *reinterpret_cast<float4 *>(s_data + k) = make_float4(0.f, 0.f, 0.f, 0.f);
  Cameras<NV> cam;
  load_cameras<S, NV>(a, t.b, t.view0, static_cast<float>(t.w) + half,
                      static_cast<float>(t.h) + half, cam);
  const S *view[NV];
  float *gview[NV];  // gradient image of the view, no lane offset
  int oy[NV], ox[NV];
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    const int64_t vo = ((int64_t)t.b * N + (t.view0 + n < N ? t.view0 + n : 0)) * view_elems;
    view[n] = a.src + vo;  // uniform: taps are addressed as base + 32-bit lane offset
    gview[n] = src_grad_img + vo;
    oy[n] = ox[n] = WN::kNone;
  }
  float tap[NV][4][VEC], sg[NV][4][VEC];
  int cur[NV];     // tap offset of the open run, -1: none
  int2 cell[NV];   // its slots and key (bit 31: inside the window)
  unsigned ring_rows[NV];  // ring rows of the window this lane's accepted cells mapped to
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    cur[n] = -1;
    ring_rows[n] = 0u;
    cell[n] = make_int2(0, 0);
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int c = 0; c < VEC; ++c) sg[n][k][c] = 0.f;
  }
  const S *cg_lane =
      CORR == 4 ? a.cost_grad + (t.pix * D * N + t.view0) * C + t.cl * VEC
                : a.cost_grad + t.pix * D * OC + (kVoxelGrad ? 0 : t.cl * (CORR ? gv : VEC));
  const int32_t *cnt_src = CORR == 4 ? a.mask_in + t.pix * D * N + t.view0
                                     : a.mask_in + t.pix * D * mask_w;
  const int32_t *mask_lane = cnt_src + t.cl * (CORR ? gv : VEC);  // this lane's part of a mask row
  // the pixel's depth gradients: the first view of a group that holds them all stores, the
  // later ones add (same lane, same address); several groups add atomically
  const bool dg_store = g.ngroups == 1 && vi == 0, dg_own = g.ngroups == 1;
  wave_sync();
  for (int d0 = d_lo; d0 < d_hi; d0 += LPP) {
    // Depth hypothesis and valid-view count of lane (p, j)'s voxel: requested before the
    // chunk's upstream-gradient rows, because loads return in order and the reprojection
    // should wait for these two words only.
    float dv = 1.f, cg_vox = 0.f;
    int cnt = REDUCE ? -1 : 0;  // "nothing to do" for a lane without a voxel
    int v3_pair = kNoPair;
    if (d0 + t.cl < d_hi) {
      dv = dv_src[d0 + t.cl];
      if (t.pix_ok) cnt = cnt_src[(int64_t)(d0 + t.cl) * cnt_step];
      if constexpr (kVoxelGrad)  // the voxel's one upstream gradient rides with its record
        cg_vox = reinterpret_cast<const float *>(cg_lane)[d0 + t.cl];
      if constexpr (CORR == 3 && REDUCE == 1) {
        if (t.pix_ok) {
          const int64_t m3 = (int64_t)(d0 + t.cl) * 3;
          const int gi = cnt_src[m3 + 1], gs = cnt_src[m3 + 2];
          // a recorded group outside the image's groups: the voxel is skipped
          if ((unsigned)gi < (unsigned)a.groups && (unsigned)gs < (unsigned)a.groups)
            v3_pair = gs * 16 + gi;
          else
            cnt = -1;
        }
      }
    }
    int r_off[NV];
    int2 r_cell[NV];
    float r_scl = 0.f;
    float4 r_wts[NV], r_dwt[NV];
    bool chunk_out[NV];  // some cell of this chunk (or the open one) sticks out of the window
    // Issue the loads of this chunk's cost_grad rows now, unconditionally, so that the
    // reprojection below overlaps their latency.  Through the caches: the workgroups of a
    // tile's views read the same rows (streamed, only about a third of the later reads found
    // them in L2).  At three waves per SIMD that was worth 2 % and cost the next forward launch
    // 5 us; at four waves it is worth 4 %, the forward launch does not notice, and 13 % less
    // is fetched.  One cache state is slower this way (by 4 %): every line dirty with another
    // kernel's output, which a load that allocates has to push out first.
    // (whole rows are kept as loaded and widened to float where a depth uses them; group
    // rows, whose width is a run-time value, are widened here and kept as float bits)
    uint32_t cgw[kVoxelGrad ? 1 : PF][(CORR == 0 || CORR == 4) ? raw_words<S, VEC>() : VEC];
    int mrow[kMaskRows ? PF : 1][VEC];
    auto load_rows = [&](int first) {
      if constexpr (CORR == 1) {
        // the group width is a run-time value: one branch around all of the chunk's loads, so
        // that they go out together (a branch per row makes each row wait for the one before)
        auto group_rows = [&](auto cnt) {
          constexpr int CNT = decltype(cnt)::value;
#pragma unroll
          for (int jj = 0; jj < PF; ++jj) {
            const int d = min(first + jj, d_hi - 1);
            load_vec<S, CNT, false>(cg_lane + (int64_t)d * cg_step, reinterpret_cast<float *>(cgw[jj]));
          }
        };
        if (g.sub == 1) group_rows(std::integral_constant<int, VEC>());
        else if (g.sub == 2) group_rows(std::integral_constant<int, VEC / 2>());
        else if (g.sub == 4) group_rows(std::integral_constant<int, VEC / 4>());
        else if constexpr (VEC >= 8) group_rows(std::integral_constant<int, VEC / 8>());
      }
#pragma unroll
      for (int jj = 0; jj < PF; ++jj) {
        const int d = min(first + jj, d_hi - 1);
        const S *src_cg = cg_lane + (int64_t)d * cg_step;
        // (each view of FeatureAggregate has rows of its own: streamed where they cover whole
        // lines)
        if constexpr (CORR == 0)
          load_raw<S, VEC, false>(src_cg, cgw[jj]);
        if constexpr (CORR == 4)
          load_raw<S, VEC, whole_lines(VEC * LPP, (int)sizeof(S))>(src_cg, cgw[jj]);
        if constexpr (kMaskRows) {
          const int32_t *m = mask_lane + (int64_t)d * OC;
          const int cntv = CORR == 0 ? VEC : gv;
          if (cntv == 4) {
            typedef int i32x4 __attribute__((ext_vector_type(4)));
            const i32x4 *q = reinterpret_cast<const i32x4 *>(m);
            const i32x4 v = *q;
            mrow[jj][0] = v[0], mrow[jj][1] = v[1], mrow[jj][2] = v[2], mrow[jj][3] = v[3];
          } else if (cntv == 2) {
            typedef int i32x2 __attribute__((ext_vector_type(2)));
            const i32x2 *q = reinterpret_cast<const i32x2 *>(m);
            const i32x2 v = *q;
            mrow[jj][0] = v[0], mrow[jj][1] = v[1];
          } else {
            mrow[jj][0] = *m;
          }
        }
      }
    };
    if constexpr (!kVoxelGrad) load_rows(d0);
    {
      const float depth = d0 + t.cl < d_hi ? (per_voxel_depth ? dv : base + dv) : 1.f;
      // factor the reduce applies to the upstream gradient: squared difference 2/k,
      // correlation 1/k, summed squared difference 2*cost_grad/(k*C) (the whole per-voxel
      // factor); zero marks a voxel that contributes nothing
      float scl = 0.f;
      if constexpr (REDUCE == 0) {
        if (cnt > 0) {
          if constexpr (CORR == 2)
            scl = 2.f * (cg_vox / static_cast<float>(cnt * C));
          else if constexpr (CORR == 3)
            scl = cg_vox / static_cast<float>(cnt);  // cost_volume_kernels_gpu_v3.cu.cc:426
          else
            scl = (CORR == 0 ? 2.f : 1.f) * __builtin_amdgcn_rcpf(static_cast<float>(cnt));
        }
      } else {
        // no division by the view count; `cnt` holds the first mask entry of the voxel (or,
        // for the summed squared difference, its winning view)
        if constexpr (CORR == 2) {
          if (cnt == t.view0) scl = 2.f * (cg_vox / static_cast<float>(C));
        } else if constexpr (CORR == 3) {
          if (cnt == t.view0) scl = cg_vox;  // cost_volume_kernels_gpu_v3.cu.cc:621-622
        } else {
          if (cnt >= 0) scl = CORR == 0 ? 2.f : 1.f;
        }
      }
#pragma unroll
      for (int n = 0; n < NV; ++n) {
        Hit hit;
        hit.off = -1;
        hit.key = 0;
        hit.k00 = hit.k01 = hit.k11 = hit.k10 = 0.f;
        float4 dw4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (t.view0 + n < N && scl != 0.f) {
          reproject<NV>(cam, n, depth, half, g.src_h_max, g.src_w_max, srcW, C, hit);
          if (DG && hit.off >= 0) {
            // d(sample)/d(depth) = sum over taps of dwt * tap, from
            //   d/d(src_h) = t1*dw + (t10 - t00),  d/d(src_w) = t1*dh + (t01 - t00),
            //   t1 = t11 - t10 - t01 + t00, chained through the perspective divide.
            const float inv = __builtin_amdgcn_rcpf(hit.z * hit.z);
            const float ah = (cam.hc[n] * hit.z - cam.zc[n] * hit.h3d) * inv;
            const float aw = (cam.wc[n] * hit.z - cam.zc[n] * hit.w3d) * inv;
            const float cp = ah * hit.dw + aw * hit.dh;
            dw4 = make_float4(cp - ah - aw, aw - cp, cp, ah - cp);  // taps 00, 01, 11, 10
          }
        }
        // The scatter window has to cover this chunk's cells and the cell still open from
        // the last chunk.  Usually it already does (one vote); otherwise it is centred on
        // their bounding box, and whatever still sticks out is marked for the memory path.
        const bool valid = hit.off >= 0;
        if (valid) {
          const unsigned fh = (unsigned)hit.key >> 16;
          ring_rows[n] |= (1u << WN::ring_row(fh)) | (1u << WN::ring_row(fh + 1u));
        }
        bool in_new = !valid || WN::inside(hit.key, oy[n], ox[n]);
        chunk_out[n] = false;
        if (__ballot(!(in_new && (cur[n] < 0 || cell[n].y < 0))) != 0ull) {
          int my = WN::kNone, mx = WN::kNone, My = -WN::kNone, Mx = -WN::kNone;
          if (valid) my = My = hit.key >> 16, mx = Mx = hit.key & 0xffff;
          if (cur[n] >= 0) {
            const int cy = (cell[n].y >> 16) & 0x7fff, cx = cell[n].y & 0xffff;
            my = min(my, cy), mx = min(mx, cx), My = max(My, cy), Mx = max(Mx, cx);
          }
          const int ny = wave_min(my), nx = wave_min(mx);
          const int hy = -wave_min(-My) + 1, hx = -wave_min(-Mx) + 1;  // last row / column used
          const int sy = WN::ROWS - (hy - ny + 1), sx = WN::COLS - (hx - nx + 1);  // slack
          window_move<VEC, LPP, kSix>(oy[n], ox[n], ny - (sy > 0 ? sy / 2 : 0),
                                nx - (sx > 0 ? sx / 2 : 0), s_data + n * WN::SLOTS * WN::STRIDE,
                                s_list, gview[n], srcW, t.lane);
          in_new = !valid || WN::inside(hit.key, oy[n], ox[n]);
          const int ck = cell[n].y & 0x7fffffff;
          cell[n].y = WN::inside(ck, oy[n], ox[n]) ? (ck | WN::kInside) : ck;
          chunk_out[n] = __ballot((valid && !in_new) || (cur[n] >= 0 && cell[n].y >= 0)) != 0ull;
        }
        const int2 rec = make_int2(WN::kPacked ? (int)WN::pack_slots(hit.key) : 0,
                                   (valid && in_new) ? (hit.key | WN::kInside) : hit.key);
        if constexpr (LPP > 1) {
          lds_at<int>(smem, q4, kOff + (n * LPP * PPW) * 4) = hit.off;
          lds_at<int2>(smem, q4 * 2u, kCell + (n * LPP * PPW) * 8) = rec;
          lds_at<float4>(smem, q4 * 4u, kWts + (n * LPP * PPW) * 16) =
              make_float4(hit.k00, hit.k01, hit.k11, hit.k10);
          if constexpr (DG) lds_at<float4>(smem, q4 * 4u, kDwt + (n * LPP * PPW) * 16) = dw4;
        } else {
          r_off[n] = hit.off;
          r_cell[n] = rec;
          r_wts[n] = make_float4(hit.k00, hit.k01, hit.k11, hit.k10);
          r_dwt[n] = dw4;
        }
      }
      if constexpr (LPP > 1) {
        lds_at<float>(smem, q4, kScl) = scl;
        if constexpr (CORR == 3)
          lds_at<int>(smem, q4, kDst) = v3_pair;  // (this op has no per-voxel depth gradient)
        else
          lds_at<float>(smem, q4, kDst) = 0.f;
      } else {
        r_scl = scl;
      }
    }
    if constexpr (LPP > 1) wave_sync();
    int rb_off[2][NV];
    float4 rb_wt[2][NV], rb_dwt[2][NV];
    float rb_scl[2];
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      if constexpr (LPP > 1) {
        rb_off[0][n] = lds_at<int>(smem, p4, kOff + (n * LPP * PPW) * 4);
        rb_wt[0][n] = lds_at<float4>(smem, p4 * 4u, kWts + (n * LPP * PPW) * 16);
        if constexpr (DG)
          rb_dwt[0][n] = lds_at<float4>(smem, p4 * 4u, kDwt + (n * LPP * PPW) * 16);
        else
          rb_dwt[0][n] = make_float4(0.f, 0.f, 0.f, 0.f);
      } else {
        rb_off[0][n] = r_off[n];
        rb_wt[0][n] = r_wts[n];
        rb_dwt[0][n] = r_dwt[n];
      }
    }
    if constexpr (LPP > 1)
      rb_scl[0] = lds_at<float>(smem, p4, kScl);
    else
      rb_scl[0] = r_scl;
#pragma unroll
    for (int jj = 0; jj < LPP; ++jj) {
      const int d = d0 + jj;
      // (no early exit past d_hi: the records of such depths carry a zero factor and no tap
      // offset, the row loads are clamped, and a loop without exits compiles to faster code)
      if constexpr (LPP > PF && !kVoxelGrad) {
        if (jj > 0 && jj % PF == 0) load_rows(d0 + jj);  // next part of a deep chunk
      }
      // The records of the NEXT depth are requested now, so that their LDS latency overlaps
      // this depth's arithmetic (jj is unrolled: the buffer index is a compile-time constant).
      // (a lean kernel reads the records of depth jj here, into the one set it keeps)
      const int cb = kLean ? 0 : (jj & 1), nb = kLean ? 0 : (cb ^ 1);
      constexpr int kAhead = kLean ? 0 : 1;
      if constexpr (LPP > 1) {
        if (kLean ? jj > 0 : jj + 1 < LPP) {
#pragma unroll
          for (int n = 0; n < NV; ++n) {
            rb_off[nb][n] = lds_at<int>(smem, p4, kOff + ((n * LPP + jj + kAhead) * PPW) * 4);
            rb_wt[nb][n] = lds_at<float4>(smem, p4 * 4u, kWts + ((n * LPP + jj + kAhead) * PPW) * 16);
            if constexpr (DG)
              rb_dwt[nb][n] = lds_at<float4>(smem, p4 * 4u, kDwt + ((n * LPP + jj + kAhead) * PPW) * 16);
            else
              rb_dwt[nb][n] = make_float4(0.f, 0.f, 0.f, 0.f);
          }
          rb_scl[nb] = lds_at<float>(smem, p4, kScl + ((jj + kAhead) * PPW) * 4);
        }
      }
      const int *rec_off = rb_off[cb];
      const float4 *rec_wt = rb_wt[cb], *rec_dwt = rb_dwt[cb];
      const float scl = rb_scl[cb];
      float dvox = 0.f;  // this lane's share of d(loss)/d(depth of this voxel)
#pragma unroll
      for (int n = 0; n < NV; ++n) {
        if (chunk_out[n]) {  // uniform, and false for the whole chunk in the usual case
          // runs that end at this depth on a cell outside the window: to memory, now
          const bool fire_out = scl != 0.f && rec_off[n] >= 0 && rec_off[n] != cur[n] &&
                                cur[n] >= 0 && cell[n].y >= 0;
          const unsigned long long m = __ballot(fire_out);
          if (m != 0ull) {
            flush_cells_to_memory<VEC, LPP>(m, fire_out, cell[n].y, sg[n], s_stage, gview[n], srcW,
                                            t.lane, t.cl);
            if (fire_out) cur[n] = -1;
          }
        }
      }
      // (one view per workgroup: a tap offset implies a non-zero factor, phase 1 reprojects
      // only voxels that have one; one test instead of two per depth)
      if (NV == 1 ? rec_off[0] >= 0 : scl != 0.f) {
        float cg[VEC];
        {
          float raw[VEC];
          if constexpr (!kVoxelGrad) {
            if (CORR == 0 || CORR == 4)
              widen_raw<S, VEC>(cgw[jj % PF], raw);
            else
#pragma unroll
              for (int c = 0; c < VEC; ++c) raw[c] = __uint_as_float(cgw[jj % PF][c]);
          }
          if constexpr (kVoxelGrad) {
#pragma unroll
            for (int c = 0; c < VEC; ++c) cg[c] = scl;
          } else if (CORR == 0 || g.sub == 1) {
#pragma unroll
            for (int c = 0; c < VEC; ++c) cg[c] = raw[c] * scl;
          } else if (g.sub == 2) {
#pragma unroll
            for (int c = 0; c < VEC; ++c) cg[c] = raw[c / 2] * scl;
          } else if (g.sub == 4) {
#pragma unroll
            for (int c = 0; c < VEC; ++c) cg[c] = raw[c / 4] * scl;
          } else {
#pragma unroll
            for (int c = 0; c < VEC; ++c) cg[c] = raw[0] * scl;
          }
          if constexpr (kMaskRows) {
            // only the channels (groups) this view won contribute
            static_assert(NV == 1, "the MIN gradient runs one view per workgroup");
            const int *mr = mrow[jj % PF];
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
              const int win = (CORR == 0 || g.sub == 1) ? mr[c]
                              : g.sub == 2              ? mr[c / 2]
                              : g.sub == 4              ? mr[c / 4]
                                                        : mr[0];
              if (win != t.view0) cg[c] = 0.f;
            }
          }
        }
#pragma unroll
        for (int n = 0; n < NV; ++n) {
          const int off = rec_off[n];
          const float4 wt = rec_wt[n], dwt = rec_dwt[n];
          if (off >= 0) {
            if (off != cur[n]) {
              // (a run whose cell sticks out of the window was closed by the uniform block
              // above, which left cur[n] = -1)
              // the run on the previous cell ends.  Start fetching the new cell's taps
              // first, then hand the old cell's image to the window while they arrive.
              // byte offsets in 32 bits: the loads take the view's base from scalar registers
              const unsigned e0 = ((unsigned)off + lane_ch) * (unsigned)sizeof(S);
              const unsigned e1 = e0 + (unsigned)row_step * (unsigned)sizeof(S);
              const char *vb = reinterpret_cast<const char *>(view[n]);
              const unsigned cb = (unsigned)C * (unsigned)sizeof(S);
              load_vec<S, VEC, false>(reinterpret_cast<const S *>(vb + e0), tap[n][0]);
              load_vec<S, VEC, false>(reinterpret_cast<const S *>(vb + (e0 + cb)), tap[n][1]);
              load_vec<S, VEC, false>(reinterpret_cast<const S *>(vb + (e1 + cb)), tap[n][2]);
              load_vec<S, VEC, false>(reinterpret_cast<const S *>(vb + e1), tap[n][3]);
              if (cur[n] >= 0)
                window_add<VEC, LPP, kLean, kSix>((unsigned)cell[n].x, cell[n].y, sg[n],
                                            s_data + n * WN::SLOTS * WN::STRIDE, s_tags, t.lane, t.cl);
              cur[n] = off;
              if constexpr (LPP > 1)
                cell[n] = lds_at<int2>(smem, p4 * 2u, kCell + ((n * LPP + jj) * PPW) * 8);
              else
                cell[n] = r_cell[n];
            }
            float gs3[VEC];
            if constexpr (CORR == 3) {
              const int pair = REDUCE ? lds_at<int>(smem, p4, kDst + (jj * PPW) * 4) : 0;
              if (g.sub == 8)
                v3_pair_gradients<VEC, LPP, 8, REDUCE>(wt, tap[n], scl, pair, s_v3, t.p, t.cl, racc,
                                                       gs3);
              else
                v3_pair_gradients<VEC, LPP, 4, REDUCE>(wt, tap[n], scl, pair, s_v3, t.p, t.cl, racc,
                                                       gs3);
            }
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
              float gsrc;  // d(loss)/d(sample of this channel)
              if constexpr (CORR == 3) {
                gsrc = gs3[c];
              } else if constexpr (CORR == 4) {
                gsrc = cg[c];
              } else if (CORR != 1) {
                float diff = __builtin_fmaf(wt.x, tap[n][0][c], -ref[c]);
                diff = __builtin_fmaf(wt.y, tap[n][1][c], diff);
                diff = __builtin_fmaf(wt.z, tap[n][2][c], diff);
                diff = __builtin_fmaf(wt.w, tap[n][3][c], diff);
                gsrc = diff * cg[c];
                racc[c] -= gsrc;
              } else {
                float smp = wt.x * tap[n][0][c];
                smp = __builtin_fmaf(wt.y, tap[n][1][c], smp);
                smp = __builtin_fmaf(wt.z, tap[n][2][c], smp);
                smp = __builtin_fmaf(wt.w, tap[n][3][c], smp);
                racc[c] = __builtin_fmaf(cg[c], smp, racc[c]);
                gsrc = cg[c] * ref[c];
              }
              sg[n][0][c] = __builtin_fmaf(gsrc, wt.x, sg[n][0][c]);
              sg[n][1][c] = __builtin_fmaf(gsrc, wt.y, sg[n][1][c]);
              sg[n][2][c] = __builtin_fmaf(gsrc, wt.z, sg[n][2][c]);
              sg[n][3][c] = __builtin_fmaf(gsrc, wt.w, sg[n][3][c]);
              if constexpr (DG) {
                float ds = dwt.x * tap[n][0][c];
                ds = __builtin_fmaf(dwt.y, tap[n][1][c], ds);
                ds = __builtin_fmaf(dwt.z, tap[n][2][c], ds);
                ds = __builtin_fmaf(dwt.w, tap[n][3][c], ds);
                dvox = __builtin_fmaf(gsrc, ds, dvox);
              }
            }
          }
        }
      }
      if constexpr (!DG) {
        // no depth gradient wanted
      } else if (per_voxel_depth) {
        if constexpr (LPP > 1) {
          const float tot = group_sum<LPP>(dvox);
          if (t.cl == 0) lds_at<float>(smem, p4, kDst + (jj * PPW) * 4) = tot;
        } else {
          if (t.pix_ok) {
            if (dg_store)
              a.depth_grad[t.pix * D + d] = dvox;
            else if (dg_own)
              a.depth_grad[t.pix * D + d] += dvox;
            else
              atomic_add(a.depth_grad + t.pix * D + d, dvox);
          }
        }
      } else {
        dacc += dvox;
      }
    }
    if constexpr (LPP > 1) {
      wave_sync();
      if (DG && per_voxel_depth) {
        const int d = d0 + t.cl;
        if (d < d_hi && t.pix_ok) {
          const float tot = lds_at<float>(smem, q4, kDst);
          if (dg_store)
            a.depth_grad[t.pix * D + d] = tot;
          else if (dg_own)
            a.depth_grad[t.pix * D + d] += tot;
          else
            atomic_add(a.depth_grad + t.pix * D + d, tot);
        }
        wave_sync();
      }
    }
  }
  // the runs still open, then everything the windows hold
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    const bool out = cur[n] >= 0 && cell[n].y >= 0;
    const unsigned long long m = __ballot(out);
    if (m != 0ull)
      flush_cells_to_memory<VEC, LPP>(m, out, cell[n].y, sg[n], s_stage, gview[n], srcW, t.lane,
                                      t.cl);
    if (cur[n] >= 0 && !out)
      window_add<VEC, LPP, false, kSix>((unsigned)cell[n].x, cell[n].y, sg[n],
                           s_data + n * WN::SLOTS * WN::STRIDE, s_tags, t.lane, t.cl);
  }
  wave_sync();
#pragma unroll
  for (int n = 0; n < NV; ++n)
    window_flush_all<VEC, LPP, kSix>(oy[n], ox[n], s_data + n * WN::SLOTS * WN::STRIDE, gview[n], srcW,
                               t.lane, wave_or(ring_rows[n]));
  wave_sync();  // the next view clears the window
  }  // views of the group

  // pixel-owned gradients: one store when this workgroup saw every depth, otherwise one
  // atomic add per depth segment into the zero-filled outputs
  float *rg = kWide ? a.ref_grad_acc : reinterpret_cast<float *>(a.ref_grad);
  const bool single = g.nseg * g.ngroups == 1;
  if constexpr (CORR == 4) {
    // no reference image, no gradient for it
  } else if (single) {
    // (16-bit storage too: the finished sums go straight to the output, the fp32 image of
    // ref_grad is neither written nor narrowed afterwards)
    if (t.pix_ok) store_vec<S, VEC, false>(a.ref_grad + t.pix * C + t.cl * VEC, racc);
  } else if (t.pix_ok) {
#pragma unroll
    for (int c = 0; c < VEC; ++c) atomic_add(rg + t.pix * C + t.cl * VEC + c, racc[c]);
  }
  if (DG && !per_voxel_depth) {
    const float tot = group_sum<LPP>(dacc);
    if (t.cl == 0 && t.pix_ok) {
      if (single)
        a.depth_grad[t.pix] = tot;
      else
        atomic_add(a.depth_grad + t.pix, tot);
    }
  }
}

// ---- host side -------------------------------------------------------------------------------
// Depth segments: enough workgroups to fill 256 CUs several times over while every segment
// keeps at least 16 hypotheses for the register-resident taps to pay off.
inline int choose_segments(int64_t tiles, int64_t D, int lpp, int64_t target_units) {
  int nseg = 1;
  const int64_t min_len = lpp > 16 ? lpp : 16;
  while (nseg < 8 && tiles * nseg < target_units && D / (nseg * 2) >= min_len) nseg *= 2;
  // a problem that does not even give every SIMD one wave: shorter segments still
  const int64_t short_len = lpp > 4 ? lpp : 4;
  while (nseg < 16 && tiles * nseg < 1024 && D / (nseg * 2) >= short_len) nseg *= 2;
  return nseg;
}

template <int LPP>
inline Geometry make_geometry(int64_t B, int64_t H, int64_t W, int64_t D, int sub, int ngroups = 1,
                              int vper = 0) {
  constexpr int PPW = 64 / LPP;
  Geometry g;
  g.hw = (int)(H * W);
  if (PPW == 1) {
    g.tiles_x = (int)W;
    g.tiles_per_image = g.hw;
  } else {
    constexpr int TH = tile_rows(PPW), TW = PPW / TH;
    g.tiles_x = (int)((W + TW - 1) / TW);
    g.tiles_per_image = g.tiles_x * (int)((H + TH - 1) / TH);
  }
  const int64_t tiles = B * g.tiles_per_image;
  g.ngroups = ngroups;
  g.vper = vper;
  // twenty waves per SIMD over the launch: the tail of a launch with fewer is measurable
  g.nseg = choose_segments(tiles * ngroups, D, LPP, 256 * 4 * 20);
  const int per_seg = (int)((D + g.nseg - 1) / g.nseg);
  g.seg = ((per_seg + LPP - 1) / LPP) * LPP;
  g.nseg = (int)((D + g.seg - 1) / g.seg);
  g.total_units = tiles * g.nseg * g.ngroups;
  g.units_per_seg = (unsigned)(tiles * g.ngroups);
  // backward: runs of 32 units (the view groups of a tile are neighbours and mostly share
  // a run, hence an L2)
  g.xcd_shift = vper > 0 ? 5 : -1;
  g.units_per_xcd = (g.total_units + 7) / 8;
  const int64_t round_to = g.xcd_shift >= 0 ? (int64_t)8 << g.xcd_shift : 8;
  g.grid = g.xcd_shift >= 0 ? (g.total_units + round_to - 1) / round_to * round_to
                            : g.units_per_xcd * 8;
  g.sub = sub;
  g.src_h_max = g.src_w_max = 0.f;  // set by the launcher from the source image size
  return g;
}

template <typename S>
inline bool aligned16(const S *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

}  // namespace tiled
}  // namespace chop
