// Constant tensor of the data model: a Meta plus row-major values held as
// float64, as the reference does (include/structure/tensor/tensor.h:37).  The
// values live in shared storage so that the many by-value copies the graph ->
// flow conversion makes (reference src/worker/converter.cpp, e.g. :144, :1236)
// cost a pointer, not a 30522x768 table.
#ifndef FLUIDML_AMD_HOST_STRUCTURE_TENSOR_TENSOR_H_
#define FLUIDML_AMD_HOST_STRUCTURE_TENSOR_TENSOR_H_

#include <memory>
#include <vector>

#include "structure/tensor/meta.h"

namespace fluidml {

class Tensor {
 public:
  explicit Tensor(Meta &&meta);
  Tensor(Meta &&meta, std::vector<float64_t> &&data);
  Tensor(Type type, std::vector<int64_t> &&shape);
  Tensor(Type type, std::vector<int64_t> &&shape, std::vector<float64_t> &&data);
  const std::vector<float64_t> &Get() const;
  float64_t &Get(const std::vector<size_t> &indices);  // detaches shared storage first
  const float64_t &Get(const std::vector<size_t> &indices) const;
  const Meta &GetMeta() const;
  Type GetType() const;
  const std::vector<int64_t> &GetShape() const;
  size_t GetHashCode() const;
  friend bool operator==(const Tensor &lhs, const Tensor &rhs);
  friend bool operator!=(const Tensor &lhs, const Tensor &rhs);

  // Dense bytes of the tensor in its element type, with `layout` applied:
  // element (i0,..) of the logical tensor lands at utils::GenStrides(shape,
  // layout). This is what gets uploaded to HBM for a constant.  `gathered`
  // (FL_REF_CONSTANT_GATHERED): the reference's form instead -- byte n in
  // row-major order takes the value found at the strided position of element
  // n (reference src/worker/builder.cpp:290-297), the same only for layouts
  // whose strided numbering is its own inverse.
  std::vector<uint8_t> Pack(const std::vector<size_t> &layout, bool gathered = false) const;

 private:
  size_t Linear(const std::vector<size_t> &indices) const;
  Meta meta_;
  std::shared_ptr<std::vector<float64_t>> data_;
};

}  // namespace fluidml

#endif
