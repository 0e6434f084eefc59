// Stand-in declarations (see op.h in this directory).
#pragma once

#include "tensorflow/core/framework/op.h"

namespace tensorflow {
namespace shape_inference {

class ShapeHandle {};
class DimensionHandle {};
// a dimension or a constant, as TensorFlow's MakeShape / MakeDim accept
struct DimensionOrConstant {
  DimensionOrConstant(DimensionHandle) {}
  DimensionOrConstant(int64) {}
};

class InferenceContext {
 public:
  template <typename T>
  Status GetAttr(const char*, T*) { return Status(); }
  ShapeHandle input(int) { return ShapeHandle(); }
  Status WithRank(ShapeHandle, int, ShapeHandle*) { return Status(); }
  DimensionHandle Dim(ShapeHandle, int) { return DimensionHandle(); }
  DimensionHandle MakeDim(DimensionOrConstant) { return DimensionHandle(); }
  ShapeHandle MakeShape(std::initializer_list<DimensionOrConstant>) { return ShapeHandle(); }
  void set_output(int, ShapeHandle) {}
};

}  // namespace shape_inference
}  // namespace tensorflow
