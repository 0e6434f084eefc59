// TensorFlow-side shim: keeps the op registrations of zhuimeng999/custom_helper_op's
// cost-volume family and turns each OpKernel into a call of libchop_costvol's C ABI.
//
// No TensorFlow exists in this repository's image: here the file only passes the compiler's
// syntax and type check against stand-in headers that declare the few TensorFlow classes it
// uses (tests/test_shim_compile.py, tests/tf_stubs/).  Build it where a ROCm TensorFlow is
// installed:
//   hipcc/g++ -std=c++17 -shared -fPIC cost_volume_ops.cc -I<repo>/include \
//       $(python -c 'import tensorflow as tf; print(" ".join(tf.sysconfig.get_compile_flags()))') \
//       $(python -c 'import tensorflow as tf; print(" ".join(tf.sysconfig.get_link_flags()))') \
//       -L<repo>/custom_helper_op_amd -lchop_costvol -o _custom_helper_ops.so
//
// Drop-in contract (what must not change, with the reference lines that fix it):
//   op names, input order, attrs, outputs      custom_helper_op/cc/ops/custom_helper_ops.cc:190-307,
//                                               :311-370 (CostVolumeV3, CostVolumeGradV3),
//                                               :374-411 (CostAggregate, CostAggregateGrad),
//                                               :414-458 (FeatureAggregate, FeatureAggregateGrad)
//   output shapes [B,H,W,D,C|groups], mask      custom_helper_ops.cc:214-219, :281-286
//   validation messages and InvalidArgument     cost_volume_kernels.cc:91-106, :220-243;
//                                               cost_volume_kernels_v2.cc:93-110, :221-247
//   DEVICE_GPU kernels for float and double     cost_volume_kernels.cc:147-154, :282-289
//   gradient registered on the Python side      custom_helper_op/python/ops/custom_helper_ops.py:41-96
// The Python wrapper of the reference loads this library unchanged.
#define EIGEN_USE_GPU

#include <string>

#include "chop_costvol.h"
#include "tensorflow/core/framework/op.h"
#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/framework/shape_inference.h"

namespace tensorflow {
namespace custom_helper_op {

using shape_inference::InferenceContext;
using shape_inference::ShapeHandle;

namespace {

// cost [B,H,W,D,last], mask [B,H,W,D,1] for MEAN and [B,H,W,D,last] otherwise.
Status VolumeShapes(InferenceContext* c, int depth_input, int depth_axis, bool grouped) {
  std::string reduce_method;
  TF_RETURN_IF_ERROR(c->GetAttr("reduce_method", &reduce_method));
  ShapeHandle ref, depth;
  TF_RETURN_IF_ERROR(c->WithRank(c->input(0), 4, &ref));
  TF_RETURN_IF_ERROR(c->WithRank(c->input(depth_input), depth_axis + 1, &depth));
  shape_inference::DimensionHandle last = c->Dim(ref, 3);
  if (grouped) {
    int32 groups;
    TF_RETURN_IF_ERROR(c->GetAttr("groups", &groups));
    last = c->MakeDim(groups);
  }
  const auto d = c->Dim(depth, depth_axis);
  c->set_output(0, c->MakeShape({c->Dim(ref, 0), c->Dim(ref, 1), c->Dim(ref, 2), d, last}));
  c->set_output(1, c->MakeShape({c->Dim(ref, 0), c->Dim(ref, 1), c->Dim(ref, 2), d,
                                 reduce_method == "MEAN" ? c->MakeDim(1) : last}));
  return Status::OK();
}

Status GradShapes(InferenceContext* c) {
  for (int i = 0; i < 3; ++i) c->set_output(i, c->input(i));
  return Status::OK();
}

}  // namespace

REGISTER_OP("CostVolume")
    .Input("ref_image: dtype")
    .Input("src_images: dtype")
    .Input("base_plane: dtype")
    .Input("offsets: dtype")
    .Input("rs: dtype")
    .Input("ts: dtype")
    .Attr("dtype: {float32,float64}")
    .Attr("reduce_method: string")
    .Attr("half_centor: bool")
    .Output("cost: dtype")
    .Output("cost_mask: int32")
    .SetShapeFn([](InferenceContext* c) { return VolumeShapes(c, 3, 1, false); });

REGISTER_OP("CostVolumeGrad")
    .Input("ref_image: dtype")
    .Input("src_images: dtype")
    .Input("base_plane: dtype")
    .Input("offsets: dtype")
    .Input("rs: dtype")
    .Input("ts: dtype")
    .Input("cost_grad: dtype")
    .Input("cost_mask: int32")
    .Attr("dtype: {float32,float64}")
    .Attr("reduce_method: string")
    .Attr("half_centor: bool")
    .Output("ref_image_grad: dtype")
    .Output("src_images_grad: dtype")
    .Output("base_plane_grad: dtype")
    .SetShapeFn(GradShapes);

REGISTER_OP("CostVolumeV2")
    .Input("ref_image: dtype")
    .Input("src_images: dtype")
    .Input("depth_grid: dtype")
    .Input("rs: dtype")
    .Input("ts: dtype")
    .Attr("dtype: {float32,float64}")
    .Attr("reduce_method: string")
    .Attr("groups: int")
    .Attr("half_centor: bool")
    .Output("cost: dtype")
    .Output("cost_mask: int32")
    .SetShapeFn([](InferenceContext* c) { return VolumeShapes(c, 2, 3, true); });

REGISTER_OP("CostVolumeGradV2")
    .Input("ref_image: dtype")
    .Input("src_images: dtype")
    .Input("depth_grid: dtype")
    .Input("rs: dtype")
    .Input("ts: dtype")
    .Input("cost_grad: dtype")
    .Input("cost_mask: int32")
    .Attr("dtype: {float32,float64}")
    .Attr("reduce_method: string")
    .Attr("groups: int")
    .Attr("half_centor: bool")
    .Output("ref_image_grad: dtype")
    .Output("src_images_grad: dtype")
    .Output("base_plane_grad: dtype")
    .SetShapeFn(GradShapes);

// cost and cost_mask [B,H,W,D] (CostAggregateShapeFn, custom_helper_ops.cc:46-58)
REGISTER_OP("CostAggregate")
    .Input("ref_image: dtype")
    .Input("src_images: dtype")
    .Input("base_plane: dtype")
    .Input("offsets: dtype")
    .Input("rs: dtype")
    .Input("ts: dtype")
    .Attr("dtype: {float32,float64}")
    .Attr("reduce_method: string")
    .Attr("half_centor: bool")
    .Output("cost: dtype")
    .Output("cost_mask: int32")
    .SetShapeFn([](InferenceContext* c) {
      ShapeHandle ref, offsets;
      TF_RETURN_IF_ERROR(c->WithRank(c->input(0), 4, &ref));
      TF_RETURN_IF_ERROR(c->WithRank(c->input(3), 2, &offsets));
      const ShapeHandle out =
          c->MakeShape({c->Dim(ref, 0), c->Dim(ref, 1), c->Dim(ref, 2), c->Dim(offsets, 1)});
      c->set_output(0, out);
      c->set_output(1, out);
      return Status::OK();
    });

REGISTER_OP("CostAggregateGrad")
    .Input("ref_image: dtype")
    .Input("src_images: dtype")
    .Input("base_plane: dtype")
    .Input("offsets: dtype")
    .Input("rs: dtype")
    .Input("ts: dtype")
    .Input("cost_grad: dtype")
    .Input("cost_mask: int32")
    .Attr("dtype: {float32,float64}")
    .Attr("reduce_method: string")
    .Attr("half_centor: bool")
    .Output("ref_image_grad: dtype")
    .Output("src_images_grad: dtype")
    .Output("base_plane_grad: dtype")
    .SetShapeFn(GradShapes);

REGISTER_OP("CostVolumeV3")
    .Input("ref_image: dtype")
    .Input("src_images: dtype")
    .Input("base_plane: dtype")
    .Input("offsets: dtype")
    .Input("rs: dtype")
    .Input("ts: dtype")
    .Attr("dtype: {float32,float64}")
    .Attr("reduce_method: string")
    .Attr("groups: int")
    .Attr("half_centor: bool")
    .Output("cost: dtype")
    .Output("cost_mask: int32")
    .SetShapeFn([](InferenceContext* c) {
      std::string reduce_method;
      TF_RETURN_IF_ERROR(c->GetAttr("reduce_method", &reduce_method));
      ShapeHandle ref, offsets;
      TF_RETURN_IF_ERROR(c->WithRank(c->input(0), 4, &ref));
      TF_RETURN_IF_ERROR(c->WithRank(c->input(3), 2, &offsets));
      const auto d = c->Dim(offsets, 1);
      c->set_output(0, c->MakeShape({c->Dim(ref, 0), c->Dim(ref, 1), c->Dim(ref, 2), d, 1}));
      c->set_output(1, c->MakeShape({c->Dim(ref, 0), c->Dim(ref, 1), c->Dim(ref, 2), d,
                                     reduce_method == "MEAN" ? 1 : 3}));
      return Status::OK();
    });

REGISTER_OP("CostVolumeGradV3")
    .Input("ref_image: dtype")
    .Input("src_images: dtype")
    .Input("base_plane: dtype")
    .Input("offsets: dtype")
    .Input("rs: dtype")
    .Input("ts: dtype")
    .Input("cost_grad: dtype")
    .Input("cost_mask: int32")
    .Attr("dtype: {float32,float64}")
    .Attr("reduce_method: string")
    .Attr("groups: int")
    .Attr("half_centor: bool")
    .Output("ref_image_grad: dtype")
    .Output("src_images_grad: dtype")
    .Output("base_plane_grad: dtype")
    .SetShapeFn(GradShapes);

REGISTER_OP("FeatureAggregate")
    .Input("src_images: dtype")
    .Input("base_plane: dtype")
    .Input("offsets: dtype")
    .Input("rs: dtype")
    .Input("ts: dtype")
    .Attr("dtype: {float32,float64}")
    .Attr("half_centor: bool")
    .Output("mapped_feature: dtype")
    .Output("mapped_mask: int32")
    .SetShapeFn([](InferenceContext* c) {
      ShapeHandle src, plane, offsets;
      TF_RETURN_IF_ERROR(c->WithRank(c->input(0), 5, &src));
      TF_RETURN_IF_ERROR(c->WithRank(c->input(1), 4, &plane));
      TF_RETURN_IF_ERROR(c->WithRank(c->input(2), 2, &offsets));
      const auto b = c->Dim(src, 0), n = c->Dim(src, 1), h = c->Dim(plane, 1), w = c->Dim(plane, 2),
                 d = c->Dim(offsets, 1);
      c->set_output(0, c->MakeShape({b, h, w, d, n, c->Dim(src, 4)}));
      c->set_output(1, c->MakeShape({b, h, w, d, n, 1}));
      return Status::OK();
    });

REGISTER_OP("FeatureAggregateGrad")
    .Input("src_images: dtype")
    .Input("base_plane: dtype")
    .Input("offsets: dtype")
    .Input("rs: dtype")
    .Input("ts: dtype")
    .Input("mapped_feature_grad: dtype")
    .Input("mapped_mask: int32")
    .Attr("dtype: {float32,float64}")
    .Attr("half_centor: bool")
    .Output("src_images_grad: dtype")
    .Output("base_plane_grad: dtype")
    .SetShapeFn([](InferenceContext* c) {
      c->set_output(0, c->input(0));
      c->set_output(1, c->input(1));
      return Status::OK();
    });

#if GOOGLE_CUDA || TENSORFLOW_USE_ROCM

typedef Eigen::GpuDevice GPUDevice;

namespace {

// One overload set per element type, so the templated kernels below stay type-agnostic.
inline int Fwd(void* s, int r, int h, const int64* d, const float* a, const float* b,
               const float* c, const float* e, const float* f, const float* g, float* o,
               int32* m) {
  return chop_cost_volume_fwd_f32(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], a, b, c,
                                  e, f, g, o, m);
}
inline int Fwd(void* s, int r, int h, const int64* d, const double* a, const double* b,
               const double* c, const double* e, const double* f, const double* g, double* o,
               int32* m) {
  return chop_cost_volume_fwd_f64(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], a, b, c,
                                  e, f, g, o, m);
}
inline int Bwd(void* s, int r, int h, const int64* d, const float* a, const float* b,
               const float* c, const float* e, const float* f, const float* g, const float* cg,
               const int32* m, float* o0, float* o1, float* o2) {
  return chop_cost_volume_bwd_f32(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], a, b, c,
                                  e, f, g, cg, m, o0, o1, o2);
}
inline int Bwd(void* s, int r, int h, const int64* d, const double* a, const double* b,
               const double* c, const double* e, const double* f, const double* g,
               const double* cg, const int32* m, double* o0, double* o1, double* o2) {
  return chop_cost_volume_bwd_f64(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], a, b, c,
                                  e, f, g, cg, m, o0, o1, o2);
}
inline int FwdAgg(void* s, int r, int h, const int64* d, const float* a, const float* b,
                  const float* c, const float* e, const float* f, const float* g, float* o,
                  int32* m) {
  return chop_cost_aggregate_fwd_f32(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], a, b,
                                     c, e, f, g, o, m);
}
inline int FwdAgg(void* s, int r, int h, const int64* d, const double* a, const double* b,
                  const double* c, const double* e, const double* f, const double* g, double* o,
                  int32* m) {
  return chop_cost_aggregate_fwd_f64(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], a, b,
                                     c, e, f, g, o, m);
}
inline int BwdAgg(void* s, int r, int h, const int64* d, const float* a, const float* b,
                  const float* c, const float* e, const float* f, const float* g, const float* cg,
                  const int32* m, float* o0, float* o1, float* o2) {
  return chop_cost_aggregate_bwd_f32(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], a, b,
                                     c, e, f, g, cg, m, o0, o1, o2);
}
inline int BwdAgg(void* s, int r, int h, const int64* d, const double* a, const double* b,
                  const double* c, const double* e, const double* f, const double* g,
                  const double* cg, const int32* m, double* o0, double* o1, double* o2) {
  return chop_cost_aggregate_bwd_f64(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], a, b,
                                     c, e, f, g, cg, m, o0, o1, o2);
}
inline int FwdV2(void* s, int r, int h, const int64* d, int groups, const float* a, const float* b,
                 const float* c, const float* f, const float* g, float* o, int32* m) {
  return chop_cost_volume_v2_fwd_f32(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], groups,
                                     a, b, c, f, g, o, m);
}
inline int FwdV2(void* s, int r, int h, const int64* d, int groups, const double* a,
                 const double* b, const double* c, const double* f, const double* g, double* o,
                 int32* m) {
  return chop_cost_volume_v2_fwd_f64(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], groups,
                                     a, b, c, f, g, o, m);
}
inline int BwdV2(void* s, int r, int h, const int64* d, int groups, const float* a, const float* b,
                 const float* c, const float* f, const float* g, const float* cg, const int32* m,
                 float* o0, float* o1, float* o2) {
  return chop_cost_volume_v2_bwd_f32(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], groups,
                                     a, b, c, f, g, cg, m, o0, o1, o2);
}
inline int BwdV2(void* s, int r, int h, const int64* d, int groups, const double* a,
                 const double* b, const double* c, const double* f, const double* g,
                 const double* cg, const int32* m, double* o0, double* o1, double* o2) {
  return chop_cost_volume_v2_bwd_f64(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], groups,
                                     a, b, c, f, g, cg, m, o0, o1, o2);
}

inline int FwdV3(void* s, int r, int h, const int64* d, int groups, const float* a, const float* b,
                 const float* c, const float* e, const float* f, const float* g, float* o,
                 int32* m) {
  return chop_cost_volume_v3_fwd_f32(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], groups,
                                     a, b, c, e, f, g, o, m);
}
inline int FwdV3(void* s, int r, int h, const int64* d, int groups, const double* a,
                 const double* b, const double* c, const double* e, const double* f,
                 const double* g, double* o, int32* m) {
  return chop_cost_volume_v3_fwd_f64(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], groups,
                                     a, b, c, e, f, g, o, m);
}
inline int BwdV3(void* s, int r, int h, const int64* d, int groups, const float* a, const float* b,
                 const float* c, const float* e, const float* f, const float* g, const float* cg,
                 const int32* m, float* o0, float* o1, float* o2) {
  return chop_cost_volume_v3_bwd_f32(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], groups,
                                     a, b, c, e, f, g, cg, m, o0, o1, o2);
}
inline int BwdV3(void* s, int r, int h, const int64* d, int groups, const double* a,
                 const double* b, const double* c, const double* e, const double* f,
                 const double* g, const double* cg, const int32* m, double* o0, double* o1,
                 double* o2) {
  return chop_cost_volume_v3_bwd_f64(s, r, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], groups,
                                     a, b, c, e, f, g, cg, m, o0, o1, o2);
}
inline int FwdFeat(void* s, int h, const int64* d, const float* b, const float* c, const float* e,
                   const float* f, const float* g, float* o, int32* m) {
  return chop_feature_aggregate_fwd_f32(s, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], b, c,
                                        e, f, g, o, m);
}
inline int FwdFeat(void* s, int h, const int64* d, const double* b, const double* c,
                   const double* e, const double* f, const double* g, double* o, int32* m) {
  return chop_feature_aggregate_fwd_f64(s, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], b, c,
                                        e, f, g, o, m);
}
inline int BwdFeat(void* s, int h, const int64* d, const float* b, const float* c, const float* e,
                   const float* f, const float* g, const float* og, const int32* m, float* o0,
                   float* o1) {
  return chop_feature_aggregate_bwd_f32(s, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], b, c,
                                        e, f, g, og, m, o0, o1);
}
inline int BwdFeat(void* s, int h, const int64* d, const double* b, const double* c,
                   const double* e, const double* f, const double* g, const double* og,
                   const int32* m, double* o0, double* o1) {
  return chop_feature_aggregate_bwd_f64(s, h, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], b, c,
                                        e, f, g, og, m, o0, o1);
}

Status FromChop(int rc) {
  if (rc == CHOP_OK) return Status::OK();
  if (rc == CHOP_ERR_LAUNCH || rc == CHOP_ERR_NO_DEVICE)
    return errors::Internal("libchop_costvol: ", chop_last_error_string());
  return errors::InvalidArgument("libchop_costvol: ", chop_last_error_string());
}

// Attributes shared by the four kernels.  An unknown reduce_method is an InvalidArgument
// at kernel construction (the reference aborts the process with LOG(FATAL),
// cost_volume_kernels.cc:66-73).
struct Attrs {
  int reduce = CHOP_REDUCE_MEAN;
  bool half_centor = true;
  int groups = 1;
  void Read(OpKernelConstruction* ctx, bool grouped) {
    std::string method;
    OP_REQUIRES_OK(ctx, ctx->GetAttr("reduce_method", &method));
    OP_REQUIRES(ctx, method == "MEAN" || method == "MIN",
                errors::InvalidArgument("Invalid reduce method ", method,
                                        ". Supported types: MEAN, MIN"));
    reduce = method == "MEAN" ? CHOP_REDUCE_MEAN : CHOP_REDUCE_MIN;
    OP_REQUIRES_OK(ctx, ctx->GetAttr("half_centor", &half_centor));
    if (grouped) OP_REQUIRES_OK(ctx, ctx->GetAttr("groups", &groups));
  }
};

// The shape checks of CostVolumeOp::Compute, shared by all four kernels.
struct Shapes {
  int64 dims[8];  // B,H,W,C,D,N,srcH,srcW
  Status Check(const Tensor& ref, const Tensor& src, const Tensor& rs, const Tensor& ts) {
    if (ref.dims() != 4) return errors::InvalidArgument("ref image must have rank 4");
    const int64 B = ref.dim_size(0), H = ref.dim_size(1), W = ref.dim_size(2), C = ref.dim_size(3);
    if (src.dims() != 5 || src.dim_size(0) != B || src.dim_size(2) != H || src.dim_size(3) != W ||
        src.dim_size(4) != C)
      return errors::InvalidArgument("src_images must have rank 5, and must compate to ref_image");
    const int64 N = src.dim_size(1);
    if (rs.dims() != 4 || rs.dim_size(0) != B || rs.dim_size(1) != N || rs.dim_size(2) != 3 ||
        rs.dim_size(3) != 3)
      return errors::InvalidArgument("Rs must have rank 2, and must compate to ref_image");
    if (ts.dims() != 3 || ts.dim_size(0) != B || ts.dim_size(1) != N || ts.dim_size(2) != 3)
      return errors::InvalidArgument("Ts must have rank 2, and must compate to ref_image");
    dims[0] = B, dims[1] = H, dims[2] = W, dims[3] = C, dims[5] = N;
    dims[6] = src.dim_size(2), dims[7] = src.dim_size(3);
    return Status::OK();
  }
  Status CheckPlane(const Tensor& base_plane, const Tensor& offsets) {
    if (base_plane.dims() != 4 || base_plane.dim_size(0) != dims[0] ||
        base_plane.dim_size(1) != dims[1] || base_plane.dim_size(2) != dims[2] ||
        base_plane.dim_size(3) != 1)
      return errors::InvalidArgument("base_plane must have rank 4, and must compate to ref_image");
    if (offsets.dims() != 2 || offsets.dim_size(0) != dims[0])
      return errors::InvalidArgument("offsets must have rank 2, and must compate to ref_image");
    dims[4] = offsets.dim_size(1);
    return Status::OK();
  }
  Status CheckGrid(const Tensor& depth_grid, int groups) {
    if (depth_grid.dims() != 4 || depth_grid.dim_size(0) != dims[0] ||
        depth_grid.dim_size(1) != dims[1] || depth_grid.dim_size(2) != dims[2])
      return errors::InvalidArgument("base_plane must have rank 4, and must compate to ref_image");
    if (groups <= 0 || dims[3] % groups != 0)
      return errors::InvalidArgument("image_channels and groups_ must match");
    dims[4] = depth_grid.dim_size(3);
    return Status::OK();
  }
  // CostVolumeV3Op::Compute, cost_volume_kernels_v3.cc:111-115
  Status CheckV3Groups(int groups) {
    if (groups <= 0 || dims[3] % groups != 0)
      return errors::InvalidArgument("image_channels and groups_ must match");
    if (dims[3] / groups > 8)
      return errors::InvalidArgument("image_channels / groups_ less than MAX_SUBCHANNELS_SIZE(8)");
    return Status::OK();
  }
  // FeatureAggregateOp::Compute, feature_aggregate_kernels.cc:69-92: the output grid is
  // base_plane's, the source images keep their own size
  Status CheckFeature(const Tensor& src, const Tensor& base_plane, const Tensor& offsets,
                      const Tensor& rs, const Tensor& ts) {
    if (src.dims() != 5) return errors::InvalidArgument("src_images must have rank 5");
    const int64 B = src.dim_size(0), N = src.dim_size(1);
    if (base_plane.dims() != 4 || base_plane.dim_size(0) != B || base_plane.dim_size(3) != 1)
      return errors::InvalidArgument("base_plane must have rank 4, and must compate to ref_image");
    if (offsets.dims() != 2 || offsets.dim_size(0) != B)
      return errors::InvalidArgument("offsets must have rank 2, and must compate to ref_image");
    if (rs.dims() != 4 || rs.dim_size(0) != B || rs.dim_size(1) != N || rs.dim_size(2) != 3 ||
        rs.dim_size(3) != 3)
      return errors::InvalidArgument("Rs must have rank 2, and must compate to ref_image");
    if (ts.dims() != 3 || ts.dim_size(0) != B || ts.dim_size(1) != N || ts.dim_size(2) != 3)
      return errors::InvalidArgument("Ts must have rank 2, and must compate to ref_image");
    dims[0] = B, dims[1] = base_plane.dim_size(1), dims[2] = base_plane.dim_size(2);
    dims[3] = src.dim_size(4), dims[4] = offsets.dim_size(1), dims[5] = N;
    dims[6] = src.dim_size(2), dims[7] = src.dim_size(3);
    return Status::OK();
  }
  Status CheckUpstream(const Tensor& cost_grad, const Tensor& cost_mask, int64 last, bool mean) {
    const TensorShape want({dims[0], dims[1], dims[2], dims[4], last});
    if (cost_grad.shape() != want)
      return errors::InvalidArgument("cost_grad must have rank 5, and must compate to ref_image");
    const TensorShape want_mask({dims[0], dims[1], dims[2], dims[4], mean ? 1 : last});
    if (cost_mask.shape() != want_mask)
      return errors::InvalidArgument("cost_mask must have rank 5, and must compate to ref_image");
    return Status::OK();
  }
};

void* StreamOf(OpKernelContext* ctx) {
  return static_cast<void*>(ctx->eigen_device<GPUDevice>().stream());
}

}  // namespace

template <typename T>
class CostVolumeOp : public OpKernel {
 public:
  explicit CostVolumeOp(OpKernelConstruction* ctx) : OpKernel(ctx) { attrs_.Read(ctx, false); }
  void Compute(OpKernelContext* ctx) override {
    const Tensor &ref = ctx->input(0), &src = ctx->input(1), &plane = ctx->input(2),
                 &offsets = ctx->input(3), &rs = ctx->input(4), &ts = ctx->input(5);
    Shapes s;
    OP_REQUIRES_OK(ctx, s.Check(ref, src, rs, ts));
    OP_REQUIRES_OK(ctx, s.CheckPlane(plane, offsets));
    const int64 *d = s.dims;
    Tensor *cost = nullptr, *mask = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, TensorShape({d[0], d[1], d[2], d[4], d[3]}), &cost));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(
                            1, TensorShape({d[0], d[1], d[2], d[4],
                                            attrs_.reduce == CHOP_REDUCE_MEAN ? 1 : d[3]}), &mask));
    OP_REQUIRES_OK(ctx, FromChop(Fwd(StreamOf(ctx), attrs_.reduce, attrs_.half_centor, d,
                                     ref.flat<T>().data(), src.flat<T>().data(),
                                     plane.flat<T>().data(), offsets.flat<T>().data(),
                                     rs.flat<T>().data(), ts.flat<T>().data(),
                                     cost->flat<T>().data(), mask->flat<int32>().data())));
  }

 private:
  Attrs attrs_;
};

template <typename T>
class CostVolumeGradOp : public OpKernel {
 public:
  explicit CostVolumeGradOp(OpKernelConstruction* ctx) : OpKernel(ctx) { attrs_.Read(ctx, false); }
  void Compute(OpKernelContext* ctx) override {
    const Tensor &ref = ctx->input(0), &src = ctx->input(1), &plane = ctx->input(2),
                 &offsets = ctx->input(3), &rs = ctx->input(4), &ts = ctx->input(5),
                 &cost_grad = ctx->input(6), &cost_mask = ctx->input(7);
    Shapes s;
    OP_REQUIRES_OK(ctx, s.Check(ref, src, rs, ts));
    OP_REQUIRES_OK(ctx, s.CheckPlane(plane, offsets));
    OP_REQUIRES_OK(ctx, s.CheckUpstream(cost_grad, cost_mask, s.dims[3],
                                        attrs_.reduce == CHOP_REDUCE_MEAN));
    Tensor *g0 = nullptr, *g1 = nullptr, *g2 = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, ref.shape(), &g0));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, src.shape(), &g1));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(2, plane.shape(), &g2));
    OP_REQUIRES_OK(ctx, FromChop(Bwd(StreamOf(ctx), attrs_.reduce, attrs_.half_centor, s.dims,
                                     ref.flat<T>().data(), src.flat<T>().data(),
                                     plane.flat<T>().data(), offsets.flat<T>().data(),
                                     rs.flat<T>().data(), ts.flat<T>().data(),
                                     cost_grad.flat<T>().data(), cost_mask.flat<int32>().data(),
                                     g0->flat<T>().data(), g1->flat<T>().data(),
                                     g2->flat<T>().data())));
  }

 private:
  Attrs attrs_;
};

template <typename T>
class CostVolumeV2Op : public OpKernel {
 public:
  explicit CostVolumeV2Op(OpKernelConstruction* ctx) : OpKernel(ctx) { attrs_.Read(ctx, true); }
  void Compute(OpKernelContext* ctx) override {
    const Tensor &ref = ctx->input(0), &src = ctx->input(1), &grid = ctx->input(2),
                 &rs = ctx->input(3), &ts = ctx->input(4);
    Shapes s;
    OP_REQUIRES_OK(ctx, s.Check(ref, src, rs, ts));
    OP_REQUIRES_OK(ctx, s.CheckGrid(grid, attrs_.groups));
    const int64 *d = s.dims, G = attrs_.groups;
    Tensor *cost = nullptr, *mask = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, TensorShape({d[0], d[1], d[2], d[4], G}), &cost));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(
                            1, TensorShape({d[0], d[1], d[2], d[4],
                                            attrs_.reduce == CHOP_REDUCE_MEAN ? 1 : G}), &mask));
    OP_REQUIRES_OK(ctx, FromChop(FwdV2(StreamOf(ctx), attrs_.reduce, attrs_.half_centor, d,
                                       attrs_.groups, ref.flat<T>().data(), src.flat<T>().data(),
                                       grid.flat<T>().data(), rs.flat<T>().data(),
                                       ts.flat<T>().data(), cost->flat<T>().data(),
                                       mask->flat<int32>().data())));
  }

 private:
  Attrs attrs_;
};

template <typename T>
class CostVolumeGradV2Op : public OpKernel {
 public:
  explicit CostVolumeGradV2Op(OpKernelConstruction* ctx) : OpKernel(ctx) { attrs_.Read(ctx, true); }
  void Compute(OpKernelContext* ctx) override {
    const Tensor &ref = ctx->input(0), &src = ctx->input(1), &grid = ctx->input(2),
                 &rs = ctx->input(3), &ts = ctx->input(4), &cost_grad = ctx->input(5),
                 &cost_mask = ctx->input(6);
    Shapes s;
    OP_REQUIRES_OK(ctx, s.Check(ref, src, rs, ts));
    OP_REQUIRES_OK(ctx, s.CheckGrid(grid, attrs_.groups));
    OP_REQUIRES_OK(ctx, s.CheckUpstream(cost_grad, cost_mask, attrs_.groups,
                                        attrs_.reduce == CHOP_REDUCE_MEAN));
    Tensor *g0 = nullptr, *g1 = nullptr, *g2 = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, ref.shape(), &g0));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, src.shape(), &g1));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(2, grid.shape(), &g2));
    OP_REQUIRES_OK(ctx, FromChop(BwdV2(StreamOf(ctx), attrs_.reduce, attrs_.half_centor, s.dims,
                                       attrs_.groups, ref.flat<T>().data(), src.flat<T>().data(),
                                       grid.flat<T>().data(), rs.flat<T>().data(),
                                       ts.flat<T>().data(), cost_grad.flat<T>().data(),
                                       cost_mask.flat<int32>().data(), g0->flat<T>().data(),
                                       g1->flat<T>().data(), g2->flat<T>().data())));
  }

 private:
  Attrs attrs_;
};

// CostAggregateOp / CostAggregateGradOp (cost_aggregate_kernels.cc:58-131, :163-259)
template <typename T>
class CostAggregateOp : public OpKernel {
 public:
  explicit CostAggregateOp(OpKernelConstruction* ctx) : OpKernel(ctx) { attrs_.Read(ctx, false); }
  void Compute(OpKernelContext* ctx) override {
    const Tensor &ref = ctx->input(0), &src = ctx->input(1), &plane = ctx->input(2),
                 &offsets = ctx->input(3), &rs = ctx->input(4), &ts = ctx->input(5);
    Shapes s;
    OP_REQUIRES_OK(ctx, s.Check(ref, src, rs, ts));
    OP_REQUIRES_OK(ctx, s.CheckPlane(plane, offsets));
    const int64 *d = s.dims;
    const TensorShape out({d[0], d[1], d[2], d[4]});
    Tensor *cost = nullptr, *mask = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, out, &cost));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, out, &mask));
    OP_REQUIRES_OK(ctx, FromChop(FwdAgg(StreamOf(ctx), attrs_.reduce, attrs_.half_centor, d,
                                        ref.flat<T>().data(), src.flat<T>().data(),
                                        plane.flat<T>().data(), offsets.flat<T>().data(),
                                        rs.flat<T>().data(), ts.flat<T>().data(),
                                        cost->flat<T>().data(), mask->flat<int32>().data())));
  }

 private:
  Attrs attrs_;
};

template <typename T>
class CostAggregateGradOp : public OpKernel {
 public:
  explicit CostAggregateGradOp(OpKernelConstruction* ctx) : OpKernel(ctx) {
    attrs_.Read(ctx, false);
  }
  void Compute(OpKernelContext* ctx) override {
    const Tensor &ref = ctx->input(0), &src = ctx->input(1), &plane = ctx->input(2),
                 &offsets = ctx->input(3), &rs = ctx->input(4), &ts = ctx->input(5),
                 &cost_grad = ctx->input(6), &cost_mask = ctx->input(7);
    Shapes s;
    OP_REQUIRES_OK(ctx, s.Check(ref, src, rs, ts));
    OP_REQUIRES_OK(ctx, s.CheckPlane(plane, offsets));
    const TensorShape want({s.dims[0], s.dims[1], s.dims[2], s.dims[4]});
    OP_REQUIRES(ctx, cost_grad.shape() == want,
                errors::InvalidArgument("cost_grad must have rank 4, and must compate to ref_image"));
    OP_REQUIRES(ctx, cost_mask.shape() == want,
                errors::InvalidArgument("cost_mask must have rank 4, and must compate to ref_image"));
    Tensor *g0 = nullptr, *g1 = nullptr, *g2 = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, ref.shape(), &g0));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, src.shape(), &g1));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(2, plane.shape(), &g2));
    OP_REQUIRES_OK(ctx, FromChop(BwdAgg(StreamOf(ctx), attrs_.reduce, attrs_.half_centor, s.dims,
                                        ref.flat<T>().data(), src.flat<T>().data(),
                                        plane.flat<T>().data(), offsets.flat<T>().data(),
                                        rs.flat<T>().data(), ts.flat<T>().data(),
                                        cost_grad.flat<T>().data(), cost_mask.flat<int32>().data(),
                                        g0->flat<T>().data(), g1->flat<T>().data(),
                                        g2->flat<T>().data())));
  }

 private:
  Attrs attrs_;
};

// CostVolumeV3Op / CostVolumeGradV3Op (cost_volume_kernels_v3.cc:58-150, :192-287)
template <typename T>
class CostVolumeV3Op : public OpKernel {
 public:
  explicit CostVolumeV3Op(OpKernelConstruction* ctx) : OpKernel(ctx) { attrs_.Read(ctx, true); }
  void Compute(OpKernelContext* ctx) override {
    const Tensor &ref = ctx->input(0), &src = ctx->input(1), &plane = ctx->input(2),
                 &offsets = ctx->input(3), &rs = ctx->input(4), &ts = ctx->input(5);
    Shapes s;
    OP_REQUIRES_OK(ctx, s.Check(ref, src, rs, ts));
    OP_REQUIRES_OK(ctx, s.CheckPlane(plane, offsets));
    OP_REQUIRES_OK(ctx, s.CheckV3Groups(attrs_.groups));
    const int64* d = s.dims;
    Tensor *cost = nullptr, *mask = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, TensorShape({d[0], d[1], d[2], d[4], 1}), &cost));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(
                            1, TensorShape({d[0], d[1], d[2], d[4],
                                            attrs_.reduce == CHOP_REDUCE_MEAN ? 1 : 3}),
                            &mask));
    OP_REQUIRES_OK(ctx, FromChop(FwdV3(StreamOf(ctx), attrs_.reduce, attrs_.half_centor, d,
                                       attrs_.groups, ref.flat<T>().data(), src.flat<T>().data(),
                                       plane.flat<T>().data(), offsets.flat<T>().data(),
                                       rs.flat<T>().data(), ts.flat<T>().data(),
                                       cost->flat<T>().data(), mask->flat<int32>().data())));
  }

 private:
  Attrs attrs_;
};

template <typename T>
class CostVolumeGradV3Op : public OpKernel {
 public:
  explicit CostVolumeGradV3Op(OpKernelConstruction* ctx) : OpKernel(ctx) { attrs_.Read(ctx, true); }
  void Compute(OpKernelContext* ctx) override {
    const Tensor &ref = ctx->input(0), &src = ctx->input(1), &plane = ctx->input(2),
                 &offsets = ctx->input(3), &rs = ctx->input(4), &ts = ctx->input(5),
                 &cost_grad = ctx->input(6), &cost_mask = ctx->input(7);
    Shapes s;
    OP_REQUIRES_OK(ctx, s.Check(ref, src, rs, ts));
    OP_REQUIRES_OK(ctx, s.CheckPlane(plane, offsets));
    OP_REQUIRES_OK(ctx, s.CheckV3Groups(attrs_.groups));
    const int64* d = s.dims;
    OP_REQUIRES(ctx, cost_grad.shape() == TensorShape({d[0], d[1], d[2], d[4], 1}),
                errors::InvalidArgument("cost_grad must have rank 5, and must compate to ref_image"));
    OP_REQUIRES(ctx,
                cost_mask.shape() == TensorShape({d[0], d[1], d[2], d[4],
                                                  attrs_.reduce == CHOP_REDUCE_MEAN ? 1 : 3}),
                errors::InvalidArgument("cost_mask must have rank 5, and must compate to ref_image"));
    Tensor *g0 = nullptr, *g1 = nullptr, *g2 = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, ref.shape(), &g0));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, src.shape(), &g1));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(2, plane.shape(), &g2));
    OP_REQUIRES_OK(ctx, FromChop(BwdV3(StreamOf(ctx), attrs_.reduce, attrs_.half_centor, d,
                                       attrs_.groups, ref.flat<T>().data(), src.flat<T>().data(),
                                       plane.flat<T>().data(), offsets.flat<T>().data(),
                                       rs.flat<T>().data(), ts.flat<T>().data(),
                                       cost_grad.flat<T>().data(), cost_mask.flat<int32>().data(),
                                       g0->flat<T>().data(), g1->flat<T>().data(),
                                       g2->flat<T>().data())));
  }

 private:
  Attrs attrs_;
};

// FeatureAggregateOp / FeatureAggregateGradOp (feature_aggregate_kernels.cc:53-118, :157-236)
template <typename T>
class FeatureAggregateOp : public OpKernel {
 public:
  explicit FeatureAggregateOp(OpKernelConstruction* ctx) : OpKernel(ctx) {
    OP_REQUIRES_OK(ctx, ctx->GetAttr("half_centor", &half_centor_));
  }
  void Compute(OpKernelContext* ctx) override {
    const Tensor &src = ctx->input(0), &plane = ctx->input(1), &offsets = ctx->input(2),
                 &rs = ctx->input(3), &ts = ctx->input(4);
    Shapes s;
    OP_REQUIRES_OK(ctx, s.CheckFeature(src, plane, offsets, rs, ts));
    const int64* d = s.dims;
    Tensor *mapped = nullptr, *mask = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(
                            0, TensorShape({d[0], d[1], d[2], d[4], d[5], d[3]}), &mapped));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, TensorShape({d[0], d[1], d[2], d[4], d[5], 1}),
                                             &mask));
    OP_REQUIRES_OK(ctx, FromChop(FwdFeat(StreamOf(ctx), half_centor_, d, src.flat<T>().data(),
                                         plane.flat<T>().data(), offsets.flat<T>().data(),
                                         rs.flat<T>().data(), ts.flat<T>().data(),
                                         mapped->flat<T>().data(), mask->flat<int32>().data())));
  }

 private:
  bool half_centor_ = true;
};

template <typename T>
class FeatureAggregateGradOp : public OpKernel {
 public:
  explicit FeatureAggregateGradOp(OpKernelConstruction* ctx) : OpKernel(ctx) {
    OP_REQUIRES_OK(ctx, ctx->GetAttr("half_centor", &half_centor_));
  }
  void Compute(OpKernelContext* ctx) override {
    const Tensor &src = ctx->input(0), &plane = ctx->input(1), &offsets = ctx->input(2),
                 &rs = ctx->input(3), &ts = ctx->input(4), &grad = ctx->input(5),
                 &mask = ctx->input(6);
    Shapes s;
    OP_REQUIRES_OK(ctx, s.CheckFeature(src, plane, offsets, rs, ts));
    const int64* d = s.dims;
    OP_REQUIRES(ctx, grad.shape() == TensorShape({d[0], d[1], d[2], d[4], d[5], d[3]}),
                errors::InvalidArgument(
                    "mapped_feature_grad must have rank 6, and must compate to src_images"));
    OP_REQUIRES(ctx, mask.shape() == TensorShape({d[0], d[1], d[2], d[4], d[5], 1}),
                errors::InvalidArgument(
                    "mapped_mask must have rank 6, and must compate to src_images"));
    Tensor *g0 = nullptr, *g1 = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, src.shape(), &g0));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, plane.shape(), &g1));
    OP_REQUIRES_OK(ctx, FromChop(BwdFeat(StreamOf(ctx), half_centor_, d, src.flat<T>().data(),
                                         plane.flat<T>().data(), offsets.flat<T>().data(),
                                         rs.flat<T>().data(), ts.flat<T>().data(),
                                         grad.flat<T>().data(), mask.flat<int32>().data(),
                                         g0->flat<T>().data(), g1->flat<T>().data())));
  }

 private:
  bool half_centor_ = true;
};

#define REGISTER_CHOP(NAME, CLASS, TYPE) \
  REGISTER_KERNEL_BUILDER(Name(NAME).Device(DEVICE_GPU).TypeConstraint<TYPE>("dtype"), CLASS<TYPE>)

REGISTER_CHOP("CostVolume", CostVolumeOp, float);
REGISTER_CHOP("CostVolume", CostVolumeOp, double);
REGISTER_CHOP("CostVolumeGrad", CostVolumeGradOp, float);
REGISTER_CHOP("CostVolumeGrad", CostVolumeGradOp, double);
REGISTER_CHOP("CostVolumeV2", CostVolumeV2Op, float);
REGISTER_CHOP("CostVolumeV2", CostVolumeV2Op, double);
REGISTER_CHOP("CostVolumeGradV2", CostVolumeGradV2Op, float);
REGISTER_CHOP("CostVolumeGradV2", CostVolumeGradV2Op, double);
REGISTER_CHOP("CostAggregate", CostAggregateOp, float);
REGISTER_CHOP("CostAggregate", CostAggregateOp, double);
REGISTER_CHOP("CostAggregateGrad", CostAggregateGradOp, float);
REGISTER_CHOP("CostAggregateGrad", CostAggregateGradOp, double);
REGISTER_CHOP("CostVolumeV3", CostVolumeV3Op, float);
REGISTER_CHOP("CostVolumeV3", CostVolumeV3Op, double);
REGISTER_CHOP("CostVolumeGradV3", CostVolumeGradV3Op, float);
REGISTER_CHOP("CostVolumeGradV3", CostVolumeGradV3Op, double);
REGISTER_CHOP("FeatureAggregate", FeatureAggregateOp, float);
REGISTER_CHOP("FeatureAggregate", FeatureAggregateOp, double);
REGISTER_CHOP("FeatureAggregateGrad", FeatureAggregateGradOp, float);
REGISTER_CHOP("FeatureAggregateGrad", FeatureAggregateGradOp, double);

#undef REGISTER_CHOP

#endif  // GOOGLE_CUDA || TENSORFLOW_USE_ROCM

}  // namespace custom_helper_op
}  // namespace tensorflow
