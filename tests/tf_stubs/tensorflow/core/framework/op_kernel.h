// Stand-in declarations (see op.h in this directory).
#pragma once

#include "tensorflow/core/framework/op.h"

namespace Eigen {
struct GpuDevice {
  void* stream() const { return nullptr; }
};
}  // namespace Eigen

namespace tensorflow {

class TensorShape {
 public:
  TensorShape() {}
  TensorShape(std::initializer_list<int64>) {}
  bool operator==(const TensorShape&) const { return true; }
  bool operator!=(const TensorShape&) const { return false; }
};

template <typename T>
struct FlatStub {
  T* data() const { return nullptr; }
};

class Tensor {
 public:
  int dims() const { return 0; }
  int64 dim_size(int) const { return 0; }
  const TensorShape& shape() const { return shape_; }
  template <typename T>
  FlatStub<const T> flat() const { return FlatStub<const T>(); }
  template <typename T>
  FlatStub<T> flat() { return FlatStub<T>(); }

 private:
  TensorShape shape_;
};

class OpKernelConstruction {
 public:
  template <typename T>
  Status GetAttr(const char*, T*) const { return Status(); }
  void CtxFailure(const Status&) {}
};

class OpKernelContext {
 public:
  const Tensor& input(int) { return tensor_; }
  Status allocate_output(int, const TensorShape&, Tensor**) { return Status(); }
  template <typename D>
  const D& eigen_device() const {
    static D d;
    return d;
  }
  void CtxFailure(const Status&) {}

 private:
  Tensor tensor_;
};

class OpKernel {
 public:
  explicit OpKernel(OpKernelConstruction*) {}
  virtual ~OpKernel() {}
  virtual void Compute(OpKernelContext*) = 0;
};

#define OP_REQUIRES(CTX, EXP, STATUS) \
  do {                                \
    if (!(EXP)) {                     \
      (CTX)->CtxFailure((STATUS));    \
      return;                         \
    }                                 \
  } while (0)

#define OP_REQUIRES_OK(CTX, ...)                  \
  do {                                            \
    ::tensorflow::Status _s(__VA_ARGS__);         \
    if (!_s.ok()) {                               \
      (CTX)->CtxFailure(_s);                      \
      return;                                     \
    }                                             \
  } while (0)

constexpr const char* DEVICE_GPU = "GPU";

class KernelDefBuilder {
 public:
  explicit KernelDefBuilder(const char*) {}
  KernelDefBuilder& Device(const char*) { return *this; }
  template <typename T>
  KernelDefBuilder& TypeConstraint(const char*) { return *this; }
};
inline KernelDefBuilder Name(const char* op) { return KernelDefBuilder(op); }

// instantiates the kernel class so that its member functions are type-checked
#define REGISTER_KERNEL_BUILDER(BUILDER, ...)                                             \
  static ::tensorflow::OpKernel* TF_STUB_CONCAT(make_kernel_, __COUNTER__)(               \
      ::tensorflow::OpKernelConstruction* c) {                                            \
    (void)(BUILDER);                                                                      \
    return new __VA_ARGS__(c);                                                            \
  }

}  // namespace tensorflow
