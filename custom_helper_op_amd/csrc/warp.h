// Device-side building blocks shared by every cost-volume kernel: storage-type traits,
// the plane-sweep reprojection with its acceptance test, and float atomics.
//
// Rounding contract.  The reprojection is written in the reference's literal operand
// order (custom_helper_op/cc/kernels/cost_volume_kernels_gpu.cu.cc:83-108) and the whole
// library is compiled with -ffp-contract=off, so the compiler never fuses a multiply with
// an add here: coordinates, truncated indices and the accepted-view set are bit-identical
// in the forward kernel, the backward kernel and a plain IEEE CPU evaluation.  Fused
// multiply-adds appear only where a kernel asks for them by name (fmaf / fma).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace chop {

// ---- storage types -------------------------------------------------------------------
struct bf16_t {
  uint16_t bits;
};

template <typename S>
struct Storage;  // Real = arithmetic type, load()/store() convert

template <>
struct Storage<float> {
  using Real = float;
  static __device__ __forceinline__ float load(const float *p) { return *p; }
  static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};
template <>
struct Storage<double> {
  using Real = double;
  static __device__ __forceinline__ double load(const double *p) { return *p; }
  static __device__ __forceinline__ void store(double *p, double v) { *p = v; }
};
template <>
struct Storage<__half> {
  using Real = float;
  static __device__ __forceinline__ float load(const __half *p) { return __half2float(*p); }
  static __device__ __forceinline__ void store(__half *p, float v) { *p = __float2half_rn(v); }
};

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits) {
  return __uint_as_float(bits << 16);
}
__device__ __forceinline__ uint32_t float_to_bf16_bits(float v) {
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;  // quiet NaN
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;                  // round to nearest even
}
template <>
struct Storage<bf16_t> {
  using Real = float;
  static __device__ __forceinline__ float load(const bf16_t *p) {
    return bf16_bits_to_float(p->bits);
  }
  static __device__ __forceinline__ void store(bf16_t *p, float v) {
    p->bits = (uint16_t)float_to_bf16_bits(v);
  }
};

template <typename R>
struct Limits;
template <>
struct Limits<float> {
  static __device__ __forceinline__ float max() { return 3.402823466e+38f; }
  static __device__ __forceinline__ float min_positive() { return 1.175494351e-38f; }
};
template <>
struct Limits<double> {
  static __device__ __forceinline__ double max() { return 1.7976931348623157e+308; }
  static __device__ __forceinline__ double min_positive() { return 2.2250738585072014e-308; }
};

// ---- reprojection ----------------------------------------------------------------------
// state: 0 behind the source camera, 1 in front but not accepted, 2 accepted.
template <typename R>
struct Sample {
  int state;
  R z_coef, w_coef, h_coef;
  R z, w3d, h3d;
  R sw, sh;
  int fh, fw;
  R dh, dw;
  R k00, k01, k11, k10;  // weights of taps (fh,fw) (fh,fw+1) (fh+1,fw+1) (fh+1,fw)
};

// cam points at 12 values: the row-major 3x3 matrix followed by the translation.
// `half` is 0.5 for the half-pixel-centre convention and 0 otherwise; adding or
// subtracting an exact 0 leaves every value unchanged, so one code path serves both.
template <typename R>
__device__ __forceinline__ void project(const R *__restrict__ Rm, const R *__restrict__ t,
                                        R ref_w, R ref_h, R depth, R half, int srcH, int srcW,
                                        Sample<R> &s) {
  s.state = 0;
  s.fh = s.fw = -1;
  s.sw = s.sh = R(0);
  s.z_coef = Rm[6] * ref_w + Rm[7] * ref_h + Rm[8];
  s.z = s.z_coef * depth + t[2];
  if (s.z <= R(0)) return;  // a NaN falls through and fails the acceptance test below
  s.state = 1;
  s.w_coef = Rm[0] * ref_w + Rm[1] * ref_h + Rm[2];
  s.w3d = s.w_coef * depth + t[0];
  s.sw = s.w3d / s.z;
  s.h_coef = Rm[3] * ref_w + Rm[4] * ref_h + Rm[5];
  s.h3d = s.h_coef * depth + t[1];
  s.sh = s.h3d / s.z;
  s.sw = s.sw - half;
  s.sh = s.sh - half;
  if (s.sh > R(0) && s.sw > R(0) && s.sh < static_cast<R>(srcH - 1) &&
      s.sw < static_cast<R>(srcW - 1)) {
    s.state = 2;
    s.fh = static_cast<int>(s.sh);
    s.fw = static_cast<int>(s.sw);
    s.dh = s.sh - static_cast<R>(s.fh);
    s.dw = s.sw - static_cast<R>(s.fw);
    s.k11 = s.dh * s.dw;
    s.k10 = s.dh * (R(1) - s.dw);
    s.k00 = (R(1) - s.dh) * (R(1) - s.dw);
    s.k01 = (R(1) - s.dh) * s.dw;
  }
}

// Coefficients that turn d(sample)/d(src_h), d(sample)/d(src_w) into d/d(depth)
// (cost_volume_kernels_gpu.cu.cc:451):  depth_grad += (ch*h_grad + cw*w_grad) / (z*z).
template <typename R>
__device__ __forceinline__ R depth_chain(const Sample<R> &s, R h_grad, R w_grad) {
  return ((s.h_coef * s.z - s.z_coef * s.h3d) * h_grad +
          (s.w_coef * s.z - s.z_coef * s.w3d) * w_grad) /
         (s.z * s.z);
}

// ---- atomics ------------------------------------------------------------------------------
// Hardware floating-point add at the L2 (global_atomic_add_f32 / _f64); the destination
// is ordinary coarse-grained device memory owned by the caller.
__device__ __forceinline__ void atomic_add(float *p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_add(double *p, double v) { unsafeAtomicAdd(p, v); }

}  // namespace chop
