// Minimal stand-in declarations for the TensorFlow symbols custom_helper_op_amd/tf_shim uses.
// They exist only so that a CPU test can run the compiler's parser and type checker over the
// shim (every chop_* call is checked against include/chop_costvol.h); they implement nothing
// and prove nothing about TensorFlow's behaviour.
#pragma once

#include <cstdint>
#include <initializer_list>
#include <string>
#include <utility>

namespace tensorflow {

typedef std::int32_t int32;
typedef std::int64_t int64;

class Status {
 public:
  static Status OK() { return Status(); }
  bool ok() const { return true; }
};

namespace errors {
template <typename... A>
Status InvalidArgument(A&&...) { return Status(); }
template <typename... A>
Status Internal(A&&...) { return Status(); }
}  // namespace errors

#define TF_RETURN_IF_ERROR(...)                       \
  do {                                                \
    ::tensorflow::Status _status = (__VA_ARGS__);     \
    if (!_status.ok()) return _status;                \
  } while (0)

namespace shape_inference {
class InferenceContext;
}

class OpDefBuilderWrapper {
 public:
  explicit OpDefBuilderWrapper(const char*) {}
  OpDefBuilderWrapper& Input(const char*) { return *this; }
  OpDefBuilderWrapper& Output(const char*) { return *this; }
  OpDefBuilderWrapper& Attr(const char*) { return *this; }
  OpDefBuilderWrapper& SetShapeFn(Status (*)(shape_inference::InferenceContext*)) { return *this; }
};

#define TF_STUB_CONCAT_(a, b) a##b
#define TF_STUB_CONCAT(a, b) TF_STUB_CONCAT_(a, b)
#define REGISTER_OP(name) \
  static ::tensorflow::OpDefBuilderWrapper TF_STUB_CONCAT(register_op_, __COUNTER__) = \
      ::tensorflow::OpDefBuilderWrapper(name)

}  // namespace tensorflow
