// Meta = element type + logical shape (reference include/structure/tensor/meta.h,
// src/structure/tensor/meta.cpp).
#ifndef FLUIDML_AMD_HOST_STRUCTURE_TENSOR_META_H_
#define FLUIDML_AMD_HOST_STRUCTURE_TENSOR_META_H_

#include <cstddef>
#include <cstdint>
#include <optional>
#include <vector>

#include "utils/type.h"

namespace fluidml {

class Meta {
 public:
  Meta(Type type, std::vector<int64_t> &&shape);
  Meta(Type type, const std::vector<int64_t> &shape);
  Type GetType() const;
  const std::vector<int64_t> &GetShape() const;
  // Prepend dims of extent `value` until the rank is `size` (meta.cpp:22-30).
  Meta AlignLeftTo(size_t size, float64_t value = 1.0) const;
  size_t GetElementsNum() const;
  // Bytes of the dense tensor; independent of any layout (meta.cpp:38-40).
  size_t GetSize() const;
  // Hash over type and dims (meta.cpp:42-51); two nodes whose metas hash and
  // compare equal share one cost-table entry in the layout DP.
  size_t GetHashCode() const;
  friend bool operator==(const Meta &lhs, const Meta &rhs);
  friend bool operator!=(const Meta &lhs, const Meta &rhs);

 private:
  Type type_;
  std::vector<int64_t> shape_;
};

// NumPy broadcast of two shapes, aligned at the trailing dims (meta.cpp:59-93).
std::optional<Meta> BroadcastShape(const Meta &lhs, const Meta &rhs, Type type);
// MatMul result shape with batch broadcast (meta.cpp:95-144); nullopt when
// either rank is below 2 or the contracted extents differ.
std::optional<Meta> BroadcastMatMulShape(const Meta &lhs, const Meta &rhs, Type type);
// Resolve a single -1 in a reshape target (meta.cpp:146-173).
std::optional<Meta> ReshapeShapeInference(const Meta &shape, size_t items);

}  // namespace fluidml

#endif
