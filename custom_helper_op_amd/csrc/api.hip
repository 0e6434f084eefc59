// C ABI of libchop_costvol: argument validation, kernel-family selection, error strings.
// Validation mirrors the checks of the reference's OpKernel::Compute
// (custom_helper_op/cc/kernels/cost_volume_kernels.cc:91-106, :220-243 and
// cost_volume_kernels_v2.cc:93-110) as far as they can be expressed on raw pointers and
// sizes; it runs before any HIP call, so bad arguments are reported on any machine.
#include <atomic>
#include <cstdio>
#include <limits>
#include <string>

#include "../../include/chop_costvol.h"
#include "internal.h"

namespace chop {
namespace {

thread_local std::string g_last_error = "";
thread_local int g_kernel_family = 0;
thread_local int g_last_family = 0;
thread_local int g_last_views_per_workgroup = 0;
thread_local int g_last_backward_window = 0;
thread_local int g_backward_window = 0;  // 0: the launcher decides, 6, 8 (chop_set_backward_window)

int fail(int code, const std::string &msg) {
  g_last_error = msg;
  return code;
}

struct Dims {
  int64_t B, H, W, C, D, N, srcH, srcW;
};

bool mul_overflows(std::initializer_list<int64_t> f, int64_t *out) {
  __int128 p = 1;
  for (int64_t v : f) {
    p *= v;
    if (p > (__int128)std::numeric_limits<int64_t>::max() / 16) return true;
  }
  *out = (int64_t)p;
  return false;
}

// Returns 0 or an error code.  Sets *empty when no kernel has to run.
int check_dims(const Dims &d, int reduce, int groups, bool correlation) {
  if (d.B < 0 || d.H < 0 || d.W < 0 || d.C < 0 || d.D < 0 || d.N < 0 || d.srcH < 0 || d.srcW < 0)
    return fail(CHOP_ERR_BAD_DIMS, "negative dimension");
  const int64_t lim = std::numeric_limits<int32_t>::max();
  if (d.H > lim || d.W > lim || d.C > lim || d.D > lim || d.N > lim || d.srcH > lim ||
      d.srcW > lim || d.B > lim)
    return fail(CHOP_ERR_BAD_DIMS, "a single dimension exceeds 2^31-1");
  int64_t tmp;
  if (mul_overflows({d.B, d.H, d.W, d.D, d.C > 0 ? d.C : 1}, &tmp) ||
      mul_overflows({d.B, d.N, d.srcH, d.srcW, d.C > 0 ? d.C : 1}, &tmp))
    return fail(CHOP_ERR_BAD_DIMS, "tensor element count overflows");
  if (reduce != CHOP_REDUCE_MEAN && reduce != CHOP_REDUCE_MIN)
    return fail(CHOP_ERR_BAD_ENUM, "reduce must be CHOP_REDUCE_MEAN (0) or CHOP_REDUCE_MIN (1)");
  if (correlation && (groups <= 0 || d.C % groups != 0))
    return fail(CHOP_ERR_BAD_GROUPS, "groups must be positive and divide the channel count");
  return 0;
}

#define REQUIRE_PTR(p, count)                                                          \
  do {                                                                                 \
    if ((p) == nullptr && (count) > 0)                                                 \
      return fail(CHOP_ERR_NULL_POINTER, std::string("null pointer: ") + #p);          \
  } while (0)

int launch_status(hipError_t err, const char *what) {
  if (err == hipSuccess) return CHOP_OK;
  return fail(CHOP_ERR_LAUNCH, std::string(what) + ": " + hipGetErrorString(err));
}

template <typename S>
int forward(void *stream, int reduce, int half_centor, const Dims &d, int groups, int corr,
            const S *ref, const S *src, const typename Storage<S>::Real *base_plane,
            const typename Storage<S>::Real *offsets, const typename Storage<S>::Real *depth_grid,
            const typename Storage<S>::Real *Rs, const typename Storage<S>::Real *Ts, S *cost,
            int32_t *mask, bool needs_depth_grid,
            const typename Storage<S>::Real *default_cost = nullptr, bool needs_default = false) {
  using R = typename Storage<S>::Real;
  if (int rc = check_dims(d, reduce, groups, corr == GROUP_CORRELATION)) return rc;
  const int64_t pixels = d.B * d.H * d.W, voxels = pixels * d.D;
  const int64_t oc = corr == GROUP_CORRELATION ? groups : d.C;
  if (voxels == 0 || oc == 0) return CHOP_OK;  // nothing to write
  REQUIRE_PTR(ref, pixels * d.C);
  REQUIRE_PTR(src, d.B * d.N * d.srcH * d.srcW * d.C);
  if (needs_depth_grid || depth_grid != nullptr) {
    REQUIRE_PTR(depth_grid, voxels);
  } else {
    REQUIRE_PTR(base_plane, pixels);
    REQUIRE_PTR(offsets, d.B * d.D);
  }
  REQUIRE_PTR(Rs, d.B * d.N);
  REQUIRE_PTR(Ts, d.B * d.N);
  REQUIRE_PTR(cost, voxels);
  REQUIRE_PTR(mask, voxels);
  if (needs_default) REQUIRE_PTR(default_cost, voxels);
  Args<S> a{};
  a.B = d.B, a.H = d.H, a.W = d.W, a.C = d.C, a.D = d.D, a.N = d.N, a.srcH = d.srcH, a.srcW = d.srcW;
  a.groups = corr == GROUP_CORRELATION ? groups : 1;
  a.reduce = reduce, a.corr = corr, a.half = half_centor ? R(0.5) : R(0);
  a.ref = ref, a.src = src, a.base_plane = base_plane, a.offsets = offsets;
  a.depth_grid = depth_grid, a.Rs = Rs, a.Ts = Ts, a.cost = cost, a.mask = mask;
  a.default_cost = default_cost;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (g_kernel_family == 0 && tiled_forward_supported(a)) {
    g_last_family = 2;
    return launch_status(launch_tiled_forward(a, s), "tiled forward launch");
  }
  if (g_kernel_family != 1 && strip_supported(a)) {
    g_last_family = 3;
    return launch_status(launch_strip_forward(a, s), "strip forward launch");
  }
  g_last_family = 1;
  return launch_status(launch_general_forward(a, s), "general forward launch");
}

template <typename S>
int backward(void *stream, int reduce, int half_centor, const Dims &d, int groups, int corr,
             const S *ref, const S *src, const typename Storage<S>::Real *base_plane,
             const typename Storage<S>::Real *offsets,
             const typename Storage<S>::Real *depth_grid, const typename Storage<S>::Real *Rs,
             const typename Storage<S>::Real *Ts, const S *cost_grad, const int32_t *mask,
             S *ref_grad, S *src_grad, typename Storage<S>::Real *depth_grad,
             bool needs_depth_grid, void *workspace, size_t workspace_bytes) {
  using R = typename Storage<S>::Real;
  if (int rc = check_dims(d, reduce, groups, corr == GROUP_CORRELATION)) return rc;
  const int64_t pixels = d.B * d.H * d.W, voxels = pixels * d.D;
  const int64_t n_ref = pixels * d.C, n_src = d.B * d.N * d.srcH * d.srcW * d.C;
  const bool per_voxel_depth = needs_depth_grid || depth_grid != nullptr;
  const int64_t n_depth = per_voxel_depth ? voxels : pixels;
  if (n_ref == 0 && n_src == 0 && n_depth == 0) return CHOP_OK;
  REQUIRE_PTR(ref_grad, n_ref);
  REQUIRE_PTR(src_grad, n_src);
  (void)n_depth;  // depth_grad may be NULL: the depth gradient is then not computed
  const bool work = voxels > 0 && d.C > 0;
  if (work) {
    REQUIRE_PTR(ref, n_ref);
    REQUIRE_PTR(src, n_src);
    if (per_voxel_depth) {
      REQUIRE_PTR(depth_grid, voxels);
    } else {
      REQUIRE_PTR(base_plane, pixels);
      REQUIRE_PTR(offsets, d.B * d.D);
    }
    REQUIRE_PTR(Rs, d.B * d.N);
    REQUIRE_PTR(Ts, d.B * d.N);
    REQUIRE_PTR(cost_grad, voxels);
    REQUIRE_PTR(mask, voxels);
  }
  Args<S> a{};
  a.B = d.B, a.H = d.H, a.W = d.W, a.C = d.C, a.D = d.D, a.N = d.N, a.srcH = d.srcH, a.srcW = d.srcW;
  a.groups = corr == GROUP_CORRELATION ? groups : 1;
  a.reduce = reduce, a.corr = corr, a.half = half_centor ? R(0.5) : R(0);
  a.ref = ref, a.src = src, a.base_plane = base_plane, a.offsets = offsets;
  a.depth_grid = depth_grid, a.Rs = Rs, a.Ts = Ts;
  a.cost_grad = cost_grad, a.mask_in = mask;
  a.ref_grad = ref_grad, a.src_grad = src_grad, a.depth_grad = depth_grad;
  if (sizeof(S) == 2) {
    const size_t need = chop_cost_volume_bwd16_workspace_bytes(d.B, d.H, d.W, d.C, d.N, d.srcH, d.srcW);
    if (need > 0) {
      if (workspace == nullptr) return fail(CHOP_ERR_WORKSPACE, "workspace is null");
      if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
        return fail(CHOP_ERR_WORKSPACE, "workspace must be 256-byte aligned");
      if (workspace_bytes < need) {
        char buf[128];
        snprintf(buf, sizeof buf, "workspace too small: %zu bytes given, %zu needed",
                 workspace_bytes, need);
        return fail(CHOP_ERR_WORKSPACE, buf);
      }
    }
    a.src_grad_acc = static_cast<float *>(workspace);
    a.ref_grad_acc = a.src_grad_acc + ((n_src + 63) / 64) * 64;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (g_kernel_family == 0 && work && tiled_backward_supported(a)) {
    g_last_family = 2;
    return launch_status(launch_tiled_backward(a, s), "tiled backward launch");
  }
  if (g_kernel_family != 1 && work && strip_supported(a)) {
    g_last_family = 3;
    return launch_status(launch_strip_backward(a, s), "strip backward launch");
  }
  g_last_family = 1;
  return launch_status(launch_general_backward(a, s), "general backward launch");
}

// CostVolumeV3 (cost_volume_kernels_v3.cc:94-115): the V1 argument checks plus
// C % groups == 0 and at most kMaxSubChannels channels per group.
template <typename S>
int v3_call(void *stream, int reduce, int half_centor, const Dims &d, int groups, const S *ref,
            const S *src, const S *base_plane, const S *offsets, const S *Rs, const S *Ts,
            S *cost, int32_t *mask, const S *cost_grad, const int32_t *mask_in, S *ref_grad,
            S *src_grad, S *base_plane_grad, bool backward) {
  if (int rc = check_dims(d, reduce, groups, true)) return rc;
  if (d.C / groups > kMaxSubChannels)
    return fail(CHOP_ERR_BAD_GROUPS, "CostVolumeV3 holds at most 8 channels per group");
  const int64_t pixels = d.B * d.H * d.W, voxels = pixels * d.D;
  const int64_t n_ref = pixels * d.C, n_src = d.B * d.N * d.srcH * d.srcW * d.C;
  const bool work = voxels > 0 && d.C > 0;
  if (backward) {
    if (n_ref == 0 && n_src == 0 && pixels == 0) return CHOP_OK;
    REQUIRE_PTR(ref_grad, n_ref);
    REQUIRE_PTR(src_grad, n_src);
    REQUIRE_PTR(base_plane_grad, pixels);
  } else {
    if (voxels == 0) return CHOP_OK;
    REQUIRE_PTR(cost, voxels);
    REQUIRE_PTR(mask, voxels);
  }
  if (work || !backward) {
    REQUIRE_PTR(ref, n_ref);
    REQUIRE_PTR(src, n_src);
    REQUIRE_PTR(base_plane, pixels);
    REQUIRE_PTR(offsets, d.B * d.D);
    REQUIRE_PTR(Rs, d.B * d.N);
    REQUIRE_PTR(Ts, d.B * d.N);
    if (backward) {
      REQUIRE_PTR(cost_grad, voxels);
      REQUIRE_PTR(mask_in, voxels);
    }
  }
  Args<S> a{};
  a.B = d.B, a.H = d.H, a.W = d.W, a.C = d.C, a.D = d.D, a.N = d.N, a.srcH = d.srcH, a.srcW = d.srcW;
  a.groups = groups, a.reduce = reduce, a.corr = BEST_GROUP_PAIR, a.half = half_centor ? S(0.5) : S(0);
  a.ref = ref, a.src = src, a.base_plane = base_plane, a.offsets = offsets, a.Rs = Rs, a.Ts = Ts;
  a.cost = cost, a.mask = mask, a.cost_grad = cost_grad, a.mask_in = mask_in;
  a.ref_grad = ref_grad, a.src_grad = src_grad, a.depth_grad = base_plane_grad;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (g_kernel_family == 0 && work) {
    if constexpr (std::is_same<S, float>::value) {
      if (backward ? tiled_backward_supported(a) : tiled_forward_supported(a)) {
        g_last_family = 2;
        return backward ? launch_status(launch_tiled_backward(a, s), "tiled CostVolumeV3 backward launch")
                        : launch_status(launch_tiled_forward(a, s), "tiled CostVolumeV3 forward launch");
      }
    }
  }
  if (g_kernel_family != 1 && work && backward && strip_pair_backward_supported(a)) {
    g_last_family = 3;
    return launch_status(launch_strip_backward(a, s), "strip CostVolumeV3 backward launch");
  }
  g_last_family = 1;
  if (backward) return launch_status(launch_v3_backward(a, s), "CostVolumeV3 backward launch");
  return launch_status(launch_v3_forward(a, s), "CostVolumeV3 forward launch");
}

// FeatureAggregate (feature_aggregate_kernels.cc:69-92): the output grid H x W is
// base_plane's, the source images have their own size.
template <typename S>
int feature_call(void *stream, int half_centor, const Dims &d, const S *src, const S *base_plane,
                 const S *offsets, const S *Rs, const S *Ts, S *mapped, int32_t *mapped_mask,
                 const S *mapped_grad, const int32_t *mask_in, S *src_grad, S *base_plane_grad,
                 bool backward) {
  if (int rc = check_dims(d, CHOP_REDUCE_MEAN, 1, false)) return rc;
  int64_t tmp;
  if (mul_overflows({d.B, d.H, d.W, d.D, d.N, d.C > 0 ? d.C : 1}, &tmp))
    return fail(CHOP_ERR_BAD_DIMS, "tensor element count overflows");
  const int64_t pixels = d.B * d.H * d.W, rows = pixels * d.D * d.N;
  const int64_t n_src = d.B * d.N * d.srcH * d.srcW * d.C;
  const bool work = rows > 0 && d.C > 0;
  if (backward) {
    if (n_src == 0 && pixels == 0) return CHOP_OK;
    REQUIRE_PTR(src_grad, n_src);
    REQUIRE_PTR(base_plane_grad, pixels);
  } else {
    if (rows == 0) return CHOP_OK;
    REQUIRE_PTR(mapped, rows * d.C);
    REQUIRE_PTR(mapped_mask, rows);
  }
  if (work || !backward) {
    REQUIRE_PTR(src, n_src);
    REQUIRE_PTR(base_plane, pixels);
    REQUIRE_PTR(offsets, d.B * d.D);
    REQUIRE_PTR(Rs, d.B * d.N);
    REQUIRE_PTR(Ts, d.B * d.N);
    if (backward) {
      REQUIRE_PTR(mapped_grad, rows * d.C);
      REQUIRE_PTR(mask_in, rows);
    }
  }
  Args<S> a{};
  a.B = d.B, a.H = d.H, a.W = d.W, a.C = d.C, a.D = d.D, a.N = d.N, a.srcH = d.srcH, a.srcW = d.srcW;
  a.groups = 1, a.reduce = CHOP_REDUCE_MEAN, a.corr = WARP_ONLY, a.half = half_centor ? S(0.5) : S(0);
  a.src = src, a.base_plane = base_plane, a.offsets = offsets, a.Rs = Rs, a.Ts = Ts;
  a.cost = mapped, a.mask = mapped_mask, a.cost_grad = mapped_grad, a.mask_in = mask_in;
  a.src_grad = src_grad, a.depth_grad = base_plane_grad;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (g_kernel_family == 0 && work) {
    if (backward ? tiled_backward_supported(a) : tiled_forward_supported(a)) {
      g_last_family = 2;
      return backward ? launch_status(launch_tiled_backward(a, s), "tiled FeatureAggregate backward launch")
                      : launch_status(launch_tiled_forward(a, s), "tiled FeatureAggregate forward launch");
    }
  }
  if (g_kernel_family != 1 && work && strip_supported(a)) {
    g_last_family = 3;
    return backward ? launch_status(launch_strip_backward(a, s), "strip FeatureAggregate backward launch")
                    : launch_status(launch_strip_forward(a, s), "strip FeatureAggregate forward launch");
  }
  g_last_family = 1;
  if (backward) return launch_status(launch_feature_backward(a, s), "FeatureAggregate backward launch");
  return launch_status(launch_feature_forward(a, s), "FeatureAggregate forward launch");
}

// ---- scratch of the entry point that allocates nothing ---------------------------------------
// chop_cost_volume_bwd_16_static keeps the fp32 gradient images of the 16-bit backward in
// this array instead of a caller-supplied workspace.  Every GPU the library runs on holds its
// own copy of the array (at its own address) from the moment the code object is loaded until
// the process ends.  On the host the name `scratch` is only a handle for hipGetSymbolAddress;
// kernels, fills and copies get the per-device address that call returns.
constexpr size_t kScratchBytes = (size_t)32 << 20;  // 32 MiB per GPU
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Address of `scratch` on the current device; looked up once per device (a race between two
// first calls stores the same address twice).  Returns nullptr with *err set on failure.
void *scratch_on_current_device(hipError_t *err) {
  int dev = -1;
  *err = hipGetDevice(&dev);
  if (*err != hipSuccess) return nullptr;
  if (dev < 0 || dev >= kMaxDevices) {
    *err = hipErrorInvalidDevice;
    return nullptr;
  }
  void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    *err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (*err != hipSuccess) return nullptr;
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  return p;
}

// The address if this device's look-up has been made, else nullptr.  No runtime call besides
// hipGetDevice.
void *scratch_if_known() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  return g_scratch_ptr[dev].load(std::memory_order_acquire);
}

}  // namespace

void note_views_per_workgroup(int views) { g_last_views_per_workgroup = views; }
int backward_window_mode() { return g_backward_window; }
void note_backward_window(int rows) { g_last_backward_window = rows; }

}  // namespace chop

using namespace chop;

extern "C" {

int chop_abi_version(void) { return 1; }

int chop_last_views_per_workgroup(void) { return g_last_family == 2 ? g_last_views_per_workgroup : 0; }

int chop_init(void) {
  hipError_t err = hipSuccess;
  if (scratch_on_current_device(&err) == nullptr) {
    if (err == hipErrorNoDevice || err == hipErrorInvalidDevice)
      return fail(CHOP_ERR_NO_DEVICE, std::string("chop_init: ") + hipGetErrorString(err));
    return launch_status(err, "address of the built-in scratch");
  }
  return CHOP_OK;
}

const char *chop_last_error_string(void) { return g_last_error.c_str(); }

int chop_set_kernel_family(int family) {
  const int prev = g_kernel_family;
  g_kernel_family = family == 1 || family == 2 ? family : 0;
  return prev;
}

int chop_last_kernel_family(void) { return g_last_family; }

int chop_last_backward_window(void) { return g_last_family == 2 ? g_last_backward_window : 0; }

int chop_set_backward_window(int rows) {
  const int prev = g_backward_window;
  g_backward_window = rows == 6 || rows == 8 ? rows : 0;
  return prev;
}

#define DIMS \
  Dims { B, H, W, C, D, N, srcH, srcW }

int chop_cost_volume_fwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                             int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                             int64_t srcW, const float *ref, const float *src,
                             const float *base_plane, const float *offsets, const float *Rs,
                             const float *Ts, float *cost, int32_t *mask) {
  return forward<float>(stream, reduce, half_centor, DIMS, 1, SQUARED_DIFFERENCE, ref, src,
                        base_plane, offsets, nullptr, Rs, Ts, cost, mask, false);
}

int chop_cost_volume_fwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                             int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                             int64_t srcW, const double *ref, const double *src,
                             const double *base_plane, const double *offsets, const double *Rs,
                             const double *Ts, double *cost, int32_t *mask) {
  return forward<double>(stream, reduce, half_centor, DIMS, 1, SQUARED_DIFFERENCE, ref, src,
                         base_plane, offsets, nullptr, Rs, Ts, cost, mask, false);
}

int chop_cost_volume_bwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                             int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                             int64_t srcW, const float *ref, const float *src,
                             const float *base_plane, const float *offsets, const float *Rs,
                             const float *Ts, const float *cost_grad, const int32_t *mask,
                             float *ref_grad, float *src_grad, float *base_plane_grad) {
  return backward<float>(stream, reduce, half_centor, DIMS, 1, SQUARED_DIFFERENCE, ref, src,
                         base_plane, offsets, nullptr, Rs, Ts, cost_grad, mask, ref_grad, src_grad,
                         base_plane_grad, false, nullptr, 0);
}

int chop_cost_volume_bwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                             int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                             int64_t srcW, const double *ref, const double *src,
                             const double *base_plane, const double *offsets, const double *Rs,
                             const double *Ts, const double *cost_grad, const int32_t *mask,
                             double *ref_grad, double *src_grad, double *base_plane_grad) {
  return backward<double>(stream, reduce, half_centor, DIMS, 1, SQUARED_DIFFERENCE, ref, src,
                          base_plane, offsets, nullptr, Rs, Ts, cost_grad, mask, ref_grad,
                          src_grad, base_plane_grad, false, nullptr, 0);
}

int chop_cost_aggregate_fwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, const float *ref, const float *src,
                                const float *base_plane, const float *offsets, const float *Rs,
                                const float *Ts, float *cost, int32_t *mask) {
  return forward<float>(stream, reduce, half_centor, DIMS, 1, SUM_SQUARED_DIFFERENCE, ref, src,
                        base_plane, offsets, nullptr, Rs, Ts, cost, mask, false);
}

int chop_cost_aggregate_fwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, const double *ref, const double *src,
                                const double *base_plane, const double *offsets,
                                const double *Rs, const double *Ts, double *cost, int32_t *mask) {
  return forward<double>(stream, reduce, half_centor, DIMS, 1, SUM_SQUARED_DIFFERENCE, ref, src,
                         base_plane, offsets, nullptr, Rs, Ts, cost, mask, false);
}

int chop_cost_aggregate_bwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, const float *ref, const float *src,
                                const float *base_plane, const float *offsets, const float *Rs,
                                const float *Ts, const float *cost_grad, const int32_t *mask,
                                float *ref_grad, float *src_grad, float *base_plane_grad) {
  return backward<float>(stream, reduce, half_centor, DIMS, 1, SUM_SQUARED_DIFFERENCE, ref, src,
                         base_plane, offsets, nullptr, Rs, Ts, cost_grad, mask, ref_grad, src_grad,
                         base_plane_grad, false, nullptr, 0);
}

int chop_cost_aggregate_bwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, const double *ref, const double *src,
                                const double *base_plane, const double *offsets,
                                const double *Rs, const double *Ts, const double *cost_grad,
                                const int32_t *mask, double *ref_grad, double *src_grad,
                                double *base_plane_grad) {
  return backward<double>(stream, reduce, half_centor, DIMS, 1, SUM_SQUARED_DIFFERENCE, ref, src,
                          base_plane, offsets, nullptr, Rs, Ts, cost_grad, mask, ref_grad,
                          src_grad, base_plane_grad, false, nullptr, 0);
}

int chop_cost_volume_v2_fwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const float *ref, const float *src,
                                const float *depth_grid, const float *Rs, const float *Ts,
                                float *cost, int32_t *mask) {
  return forward<float>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION, ref, src,
                        nullptr, nullptr, depth_grid, Rs, Ts, cost, mask, true);
}

int chop_cost_volume_v2_fwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const double *ref, const double *src,
                                const double *depth_grid, const double *Rs, const double *Ts,
                                double *cost, int32_t *mask) {
  return forward<double>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION, ref, src,
                         nullptr, nullptr, depth_grid, Rs, Ts, cost, mask, true);
}

int chop_cost_volume_v2_bwd_f32(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const float *ref, const float *src,
                                const float *depth_grid, const float *Rs, const float *Ts,
                                const float *cost_grad, const int32_t *mask, float *ref_grad,
                                float *src_grad, float *depth_grid_grad) {
  return backward<float>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION, ref, src,
                         nullptr, nullptr, depth_grid, Rs, Ts, cost_grad, mask, ref_grad,
                         src_grad, depth_grid_grad, true, nullptr, 0);
}

int chop_cost_volume_v2_bwd_f64(void *stream, int reduce, int half_centor, int64_t B, int64_t H,
                                int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                                int64_t srcW, int groups, const double *ref, const double *src,
                                const double *depth_grid, const double *Rs, const double *Ts,
                                const double *cost_grad, const int32_t *mask, double *ref_grad,
                                double *src_grad, double *depth_grid_grad) {
  return backward<double>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION, ref, src,
                          nullptr, nullptr, depth_grid, Rs, Ts, cost_grad, mask, ref_grad,
                          src_grad, depth_grid_grad, true, nullptr, 0);
}

// The forward ops of the two cost-map layers with the layers' default fill folded into the
// store (custom_helper_op/python/layers/custom_layers.py:51-57, :77-83).
#define FILL_ENTRY(SFX, T)                                                                      \
  int chop_cost_aggregate_fwd_fill_##SFX(void *stream, int reduce, int half_centor, int64_t B,  \
                                         int64_t H, int64_t W, int64_t C, int64_t D, int64_t N, \
                                         int64_t srcH, int64_t srcW, const T *ref, const T *src, \
                                         const T *base_plane, const T *offsets, const T *Rs,    \
                                         const T *Ts, const T *default_cost, T *cost,           \
                                         int32_t *mask) {                                       \
    return forward<T>(stream, reduce, half_centor, DIMS, 1, SUM_SQUARED_DIFFERENCE, ref, src,   \
                      base_plane, offsets, nullptr, Rs, Ts, cost, mask, false, default_cost,    \
                      true);                                                                    \
  }                                                                                             \
  int chop_cost_volume_v2_fwd_fill_##SFX(void *stream, int reduce, int half_centor, int64_t B,  \
                                         int64_t H, int64_t W, int64_t C, int64_t D, int64_t N, \
                                         int64_t srcH, int64_t srcW, int groups, const T *ref,  \
                                         const T *src, const T *depth_grid, const T *Rs,        \
                                         const T *Ts, const T *default_cost, T *cost,           \
                                         int32_t *mask) {                                       \
    return forward<T>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION, ref, src,   \
                      nullptr, nullptr, depth_grid, Rs, Ts, cost, mask, true, default_cost,     \
                      true);                                                                    \
  }
FILL_ENTRY(f32, float)
FILL_ENTRY(f64, double)
#undef FILL_ENTRY

#define V3_ENTRY(SFX, T)                                                                       \
  int chop_cost_volume_v3_fwd_##SFX(void *stream, int reduce, int half_centor, int64_t B,      \
                                    int64_t H, int64_t W, int64_t C, int64_t D, int64_t N,     \
                                    int64_t srcH, int64_t srcW, int groups, const T *ref,      \
                                    const T *src, const T *base_plane, const T *offsets,       \
                                    const T *Rs, const T *Ts, T *cost, int32_t *mask) {        \
    return v3_call<T>(stream, reduce, half_centor, DIMS, groups, ref, src, base_plane, offsets, \
                      Rs, Ts, cost, mask, nullptr, nullptr, nullptr, nullptr, nullptr, false);  \
  }                                                                                            \
  int chop_cost_volume_v3_bwd_##SFX(void *stream, int reduce, int half_centor, int64_t B,      \
                                    int64_t H, int64_t W, int64_t C, int64_t D, int64_t N,     \
                                    int64_t srcH, int64_t srcW, int groups, const T *ref,      \
                                    const T *src, const T *base_plane, const T *offsets,       \
                                    const T *Rs, const T *Ts, const T *cost_grad,              \
                                    const int32_t *mask, T *ref_grad, T *src_grad,             \
                                    T *base_plane_grad) {                                      \
    return v3_call<T>(stream, reduce, half_centor, DIMS, groups, ref, src, base_plane, offsets, \
                      Rs, Ts, nullptr, nullptr, cost_grad, mask, ref_grad, src_grad,            \
                      base_plane_grad, true);                                                   \
  }                                                                                            \
  int chop_feature_aggregate_fwd_##SFX(void *stream, int half_centor, int64_t B, int64_t H,    \
                                       int64_t W, int64_t C, int64_t D, int64_t N,             \
                                       int64_t srcH, int64_t srcW, const T *src,               \
                                       const T *base_plane, const T *offsets, const T *Rs,     \
                                       const T *Ts, T *mapped_feature, int32_t *mapped_mask) { \
    return feature_call<T>(stream, half_centor, DIMS, src, base_plane, offsets, Rs, Ts,        \
                           mapped_feature, mapped_mask, nullptr, nullptr, nullptr, nullptr,    \
                           false);                                                             \
  }                                                                                            \
  int chop_feature_aggregate_bwd_##SFX(void *stream, int half_centor, int64_t B, int64_t H,    \
                                       int64_t W, int64_t C, int64_t D, int64_t N,             \
                                       int64_t srcH, int64_t srcW, const T *src,               \
                                       const T *base_plane, const T *offsets, const T *Rs,     \
                                       const T *Ts, const T *mapped_feature_grad,              \
                                       const int32_t *mapped_mask, T *src_grad,                \
                                       T *base_plane_grad) {                                   \
    return feature_call<T>(stream, half_centor, DIMS, src, base_plane, offsets, Rs, Ts,        \
                           nullptr, nullptr, mapped_feature_grad, mapped_mask, src_grad,       \
                           base_plane_grad, true);                                             \
  }
V3_ENTRY(f32, float)
V3_ENTRY(f64, double)
#undef V3_ENTRY

#define EPILOGUE_ENTRY(SFX, T)                                                                  \
  int chop_cost_default_fill_##SFX(void *stream, int reduce, int64_t mask_count, int64_t inner, \
                                   const T *cost, const int32_t *mask, const T *default_cost,   \
                                   T *out) {                                                    \
    if (reduce != CHOP_REDUCE_MEAN && reduce != CHOP_REDUCE_MIN)                                \
      return fail(CHOP_ERR_BAD_ENUM, "reduce must be CHOP_REDUCE_MEAN (0) or CHOP_REDUCE_MIN (1)"); \
    int64_t total;                                                                              \
    if (mask_count < 0 || inner < 1 || mul_overflows({mask_count, inner}, &total))              \
      return fail(CHOP_ERR_BAD_DIMS, "mask_count must be >= 0 and inner >= 1");                 \
    if (total == 0) return CHOP_OK;                                                             \
    REQUIRE_PTR(cost, total);                                                                   \
    REQUIRE_PTR(mask, total);                                                                   \
    REQUIRE_PTR(default_cost, total);                                                           \
    REQUIRE_PTR(out, total);                                                                    \
    return launch_status(launch_default_fill<T>(reduce, mask_count, inner, cost, mask,          \
                                                default_cost, out,                              \
                                                static_cast<hipStream_t>(stream)),              \
                         "default fill launch");                                                \
  }                                                                                             \
  int chop_cost_default_fill_grad_##SFX(void *stream, int reduce, int64_t mask_count,           \
                                        int64_t inner, const T *out_grad, const int32_t *mask,  \
                                        T *cost_grad, T *default_grad) {                        \
    if (reduce != CHOP_REDUCE_MEAN && reduce != CHOP_REDUCE_MIN)                                \
      return fail(CHOP_ERR_BAD_ENUM, "reduce must be CHOP_REDUCE_MEAN (0) or CHOP_REDUCE_MIN (1)"); \
    int64_t total;                                                                              \
    if (mask_count < 0 || inner < 1 || mul_overflows({mask_count, inner}, &total))              \
      return fail(CHOP_ERR_BAD_DIMS, "mask_count must be >= 0 and inner >= 1");                 \
    REQUIRE_PTR(default_grad, 1);                                                               \
    REQUIRE_PTR(out_grad, total);                                                               \
    REQUIRE_PTR(mask, total);                                                                   \
    return launch_status(launch_default_fill_grad<T>(reduce, mask_count, inner, out_grad, mask, \
                                                     cost_grad, default_grad,                   \
                                                     static_cast<hipStream_t>(stream)),         \
                         "default fill gradient launch");                                       \
  }                                                                                             \
  int chop_combine_projection_##SFX(void *stream, int64_t B, int64_t N, const T *ref_cam,       \
                                    const T *src_cam, const T *scale, T *Rs, T *Ts) {           \
    int64_t total;                                                                              \
    if (B < 0 || N < 0 || mul_overflows({B, N, 32}, &total))                                    \
      return fail(CHOP_ERR_BAD_DIMS, "B and N must be >= 0");                                   \
    if (total == 0) return CHOP_OK;                                                             \
    REQUIRE_PTR(ref_cam, total);                                                                \
    REQUIRE_PTR(src_cam, total);                                                                \
    REQUIRE_PTR(scale, total);                                                                  \
    REQUIRE_PTR(Rs, total);                                                                     \
    REQUIRE_PTR(Ts, total);                                                                     \
    return launch_status(launch_combine_projection<T>(B, N, ref_cam, src_cam, scale, Rs, Ts,    \
                                                      static_cast<hipStream_t>(stream)),        \
                         "combine_projection launch");                                          \
  }
EPILOGUE_ENTRY(f32, float)
EPILOGUE_ENTRY(f64, double)
#undef EPILOGUE_ENTRY

size_t chop_cost_volume_bwd16_workspace_bytes(int64_t B, int64_t H, int64_t W, int64_t C,
                                              int64_t N, int64_t srcH, int64_t srcW) {
  if (B < 0 || H < 0 || W < 0 || C < 0 || N < 0 || srcH < 0 || srcW < 0) return 0;
  const int64_t n_src = B * N * srcH * srcW * C, n_ref = B * H * W * C;
  return (size_t)(((n_src + 63) / 64) * 64 + ((n_ref + 63) / 64) * 64) * sizeof(float);
}

#define STORAGE_DISPATCH(expr_half, expr_bf16)                                              \
  switch (storage) {                                                                        \
    case CHOP_STORAGE_F16:                                                                  \
      return expr_half;                                                                     \
    case CHOP_STORAGE_BF16:                                                                 \
      return expr_bf16;                                                                     \
    default:                                                                                \
      return fail(CHOP_ERR_BAD_ENUM, "storage must be CHOP_STORAGE_F16 or CHOP_STORAGE_BF16"); \
  }

int chop_cost_volume_fwd_16(void *stream, int storage, int reduce, int half_centor, int64_t B,
                            int64_t H, int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                            int64_t srcW, const void *ref, const void *src,
                            const float *base_plane, const float *offsets,
                            const float *depth_grid, const float *Rs, const float *Ts,
                            void *cost, int32_t *mask) {
  STORAGE_DISPATCH(
      forward<__half>(stream, reduce, half_centor, DIMS, 1, SQUARED_DIFFERENCE,
                      (const __half *)ref, (const __half *)src, base_plane, offsets, depth_grid,
                      Rs, Ts, (__half *)cost, mask, false),
      forward<bf16_t>(stream, reduce, half_centor, DIMS, 1, SQUARED_DIFFERENCE,
                      (const bf16_t *)ref, (const bf16_t *)src, base_plane, offsets, depth_grid,
                      Rs, Ts, (bf16_t *)cost, mask, false))
}

int chop_cost_volume_bwd_16(void *stream, int storage, int reduce, int half_centor, int64_t B,
                            int64_t H, int64_t W, int64_t C, int64_t D, int64_t N, int64_t srcH,
                            int64_t srcW, const void *ref, const void *src,
                            const float *base_plane, const float *offsets,
                            const float *depth_grid, const float *Rs, const float *Ts,
                            const void *cost_grad, const int32_t *mask, void *ref_grad,
                            void *src_grad, float *depth_grad, void *workspace,
                            size_t workspace_bytes) {
  STORAGE_DISPATCH(
      backward<__half>(stream, reduce, half_centor, DIMS, 1, SQUARED_DIFFERENCE,
                       (const __half *)ref, (const __half *)src, base_plane, offsets, depth_grid,
                       Rs, Ts, (const __half *)cost_grad, mask, (__half *)ref_grad,
                       (__half *)src_grad, depth_grad, false, workspace, workspace_bytes),
      backward<bf16_t>(stream, reduce, half_centor, DIMS, 1, SQUARED_DIFFERENCE,
                       (const bf16_t *)ref, (const bf16_t *)src, base_plane, offsets, depth_grid,
                       Rs, Ts, (const bf16_t *)cost_grad, mask, (bf16_t *)ref_grad,
                       (bf16_t *)src_grad, depth_grad, false, workspace, workspace_bytes))
}

int chop_cost_default_fill_grad_16(void *stream, int storage, int reduce, int64_t mask_count,
                                   int64_t inner, const void *out_grad, const int32_t *mask,
                                   void *cost_grad, float *default_grad) {
  if (reduce != CHOP_REDUCE_MEAN && reduce != CHOP_REDUCE_MIN)
    return fail(CHOP_ERR_BAD_ENUM, "reduce must be CHOP_REDUCE_MEAN (0) or CHOP_REDUCE_MIN (1)");
  int64_t total;
  if (mask_count < 0 || inner < 1 || mul_overflows({mask_count, inner}, &total))
    return fail(CHOP_ERR_BAD_DIMS, "mask_count must be >= 0 and inner >= 1");
  REQUIRE_PTR(default_grad, 1);
  REQUIRE_PTR(out_grad, total);
  REQUIRE_PTR(mask, total);
  hipStream_t s = static_cast<hipStream_t>(stream);
  STORAGE_DISPATCH(
      launch_status(launch_default_fill_grad<__half>(reduce, mask_count, inner,
                                                     (const __half *)out_grad, mask,
                                                     (__half *)cost_grad, default_grad, s),
                    "default fill gradient launch"),
      launch_status(launch_default_fill_grad<bf16_t>(reduce, mask_count, inner,
                                                     (const bf16_t *)out_grad, mask,
                                                     (bf16_t *)cost_grad, default_grad, s),
                    "default fill gradient launch"))
}

size_t chop_static_scratch_bytes(void) { return kScratchBytes; }

int chop_cost_volume_bwd_16_static(void *stream, int storage, int reduce, int half_centor,
                                   int64_t B, int64_t H, int64_t W, int64_t C, int64_t D,
                                   int64_t N, int64_t srcH, int64_t srcW, const void *ref,
                                   const void *src, const float *base_plane,
                                   const float *offsets, const float *depth_grid,
                                   const float *Rs, const float *Ts, const void *cost_grad,
                                   const int32_t *mask, void *ref_grad, void *src_grad,
                                   float *depth_grad) {
  const size_t need = chop_cost_volume_bwd16_workspace_bytes(B, H, W, C, N, srcH, srcW);
  if (need > kScratchBytes) {
    char buf[192];
    snprintf(buf, sizeof buf,
             "the gradient images need %zu bytes, the built-in scratch holds %zu: use "
             "chop_cost_volume_bwd_16 with a workspace of the caller",
             need, kScratchBytes);
    return fail(CHOP_ERR_WORKSPACE, buf);
  }
  hipError_t err = hipSuccess;
  void *ws = scratch_if_known();
  if (ws == nullptr) {
    // first use on this device.  The look-up is a runtime query, not stream work: it does
    // not belong inside a capture, so a capturing caller has to have made it before
    // (chop_init, or any earlier call of this entry point on the device).
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &cap) == hipSuccess &&
        cap != hipStreamCaptureStatusNone)
      return fail(CHOP_ERR_WORKSPACE,
                  "the built-in scratch has not been located on this device yet: call "
                  "chop_init() once per device before capturing");
    ws = scratch_on_current_device(&err);
    if (ws == nullptr) return launch_status(err, "address of the built-in scratch");
  }
  // (the launch clears the part of the scratch it accumulates into: launch_tiled_backward /
  // launch_general_backward zero-fill both gradient images with a kernel before they add)
  return chop_cost_volume_bwd_16(stream, storage, reduce, half_centor, B, H, W, C, D, N, srcH,
                                 srcW, ref, src, base_plane, offsets, depth_grid, Rs, Ts,
                                 cost_grad, mask, ref_grad, src_grad, depth_grad, ws,
                                 kScratchBytes);
}

int chop_cost_volume_v2_fwd_16(void *stream, int storage, int reduce, int half_centor, int64_t B,
                               int64_t H, int64_t W, int64_t C, int64_t D, int64_t N,
                               int64_t srcH, int64_t srcW, int groups, const void *ref,
                               const void *src, const float *depth_grid, const float *Rs,
                               const float *Ts, void *cost, int32_t *mask) {
  STORAGE_DISPATCH(
      forward<__half>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION,
                      (const __half *)ref, (const __half *)src, nullptr, nullptr, depth_grid, Rs,
                      Ts, (__half *)cost, mask, true),
      forward<bf16_t>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION,
                      (const bf16_t *)ref, (const bf16_t *)src, nullptr, nullptr, depth_grid, Rs,
                      Ts, (bf16_t *)cost, mask, true))
}

int chop_cost_volume_v2_fwd_fill_16(void *stream, int storage, int reduce, int half_centor,
                                    int64_t B, int64_t H, int64_t W, int64_t C, int64_t D,
                                    int64_t N, int64_t srcH, int64_t srcW, int groups,
                                    const void *ref, const void *src, const float *depth_grid,
                                    const float *Rs, const float *Ts, const float *default_cost,
                                    void *cost, int32_t *mask) {
  STORAGE_DISPATCH(
      forward<__half>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION,
                      (const __half *)ref, (const __half *)src, nullptr, nullptr, depth_grid, Rs,
                      Ts, (__half *)cost, mask, true, default_cost, true),
      forward<bf16_t>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION,
                      (const bf16_t *)ref, (const bf16_t *)src, nullptr, nullptr, depth_grid, Rs,
                      Ts, (bf16_t *)cost, mask, true, default_cost, true))
}

int chop_cost_volume_v2_bwd_16(void *stream, int storage, int reduce, int half_centor, int64_t B,
                               int64_t H, int64_t W, int64_t C, int64_t D, int64_t N,
                               int64_t srcH, int64_t srcW, int groups, const void *ref,
                               const void *src, const float *depth_grid, const float *Rs,
                               const float *Ts, const void *cost_grad, const int32_t *mask,
                               void *ref_grad, void *src_grad, float *depth_grid_grad,
                               void *workspace, size_t workspace_bytes) {
  STORAGE_DISPATCH(
      backward<__half>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION,
                       (const __half *)ref, (const __half *)src, nullptr, nullptr, depth_grid, Rs,
                       Ts, (const __half *)cost_grad, mask, (__half *)ref_grad,
                       (__half *)src_grad, depth_grid_grad, true, workspace, workspace_bytes),
      backward<bf16_t>(stream, reduce, half_centor, DIMS, groups, GROUP_CORRELATION,
                       (const bf16_t *)ref, (const bf16_t *)src, nullptr, nullptr, depth_grid, Rs,
                       Ts, (const bf16_t *)cost_grad, mask, (bf16_t *)ref_grad,
                       (bf16_t *)src_grad, depth_grid_grad, true, workspace, workspace_bytes))
}

int chop_cost_volume_sample_coords_f32(void *stream, int half_centor, int64_t B, int64_t H,
                                       int64_t W, int64_t D, int64_t N, int64_t srcH,
                                       int64_t srcW, const float *base_plane,
                                       const float *offsets, const float *depth_grid,
                                       const float *Rs, const float *Ts, float *sw, float *sh,
                                       int32_t *fh, int32_t *fw, int32_t *state) {
  const Dims d{B, H, W, 1, D, N, srcH, srcW};
  if (int rc = check_dims(d, 0, 1, false)) return rc;
  const int64_t total = B * H * W * D * N;
  if (total == 0) return CHOP_OK;
  if (depth_grid == nullptr) {
    REQUIRE_PTR(base_plane, total);
    REQUIRE_PTR(offsets, total);
  }
  REQUIRE_PTR(Rs, total); REQUIRE_PTR(Ts, total); REQUIRE_PTR(sw, total); REQUIRE_PTR(sh, total);
  REQUIRE_PTR(fh, total); REQUIRE_PTR(fw, total); REQUIRE_PTR(state, total);
  return launch_status(
      launch_sample_coords<float>(half_centor ? 0.5f : 0.f, B, H, W, D, N, srcH, srcW, base_plane,
                                  offsets, depth_grid, Rs, Ts, sw, sh, fh, fw, state,
                                  static_cast<hipStream_t>(stream)),
      "sample_coords launch");
}

int chop_cost_volume_sample_coords_f64(void *stream, int half_centor, int64_t B, int64_t H,
                                       int64_t W, int64_t D, int64_t N, int64_t srcH,
                                       int64_t srcW, const double *base_plane,
                                       const double *offsets, const double *depth_grid,
                                       const double *Rs, const double *Ts, double *sw,
                                       double *sh, int32_t *fh, int32_t *fw, int32_t *state) {
  const Dims d{B, H, W, 1, D, N, srcH, srcW};
  if (int rc = check_dims(d, 0, 1, false)) return rc;
  const int64_t total = B * H * W * D * N;
  if (total == 0) return CHOP_OK;
  if (depth_grid == nullptr) {
    REQUIRE_PTR(base_plane, total);
    REQUIRE_PTR(offsets, total);
  }
  REQUIRE_PTR(Rs, total); REQUIRE_PTR(Ts, total); REQUIRE_PTR(sw, total); REQUIRE_PTR(sh, total);
  REQUIRE_PTR(fh, total); REQUIRE_PTR(fw, total); REQUIRE_PTR(state, total);
  return launch_status(
      launch_sample_coords<double>(half_centor ? 0.5 : 0.0, B, H, W, D, N, srcH, srcW, base_plane,
                                   offsets, depth_grid, Rs, Ts, sw, sh, fh, fw, state,
                                   static_cast<hipStream_t>(stream)),
      "sample_coords launch");
}

}  // extern "C"
