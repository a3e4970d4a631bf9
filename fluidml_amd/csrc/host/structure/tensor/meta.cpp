#include "structure/tensor/meta.h"

#include <algorithm>
#include <functional>

namespace fluidml {

namespace {
// hash ^= h(x) + seed + (hash << 6) + (hash >> 2) with seed 0, as the
// reference combines (include/utils/hash.h:8, meta.cpp:47-49)
inline void Combine(size_t &hash, size_t value) { hash ^= value + 0 + (hash << 6) + (hash >> 2); }

std::optional<std::vector<int64_t>> BroadcastDims(const std::vector<int64_t> &lhs, const std::vector<int64_t> &rhs,
                                                  size_t count) {
  std::vector<int64_t> out(count);
  for (size_t i = 0; i < count; ++i) {
    if (lhs[i] == rhs[i] || rhs[i] == 1) {
      out[i] = lhs[i];
    } else if (lhs[i] == 1) {
      out[i] = rhs[i];
    } else {
      return std::nullopt;
    }
  }
  return out;
}
}  // namespace

Meta::Meta(Type type, std::vector<int64_t> &&shape) : type_(type), shape_(std::move(shape)) {}
Meta::Meta(Type type, const std::vector<int64_t> &shape) : type_(type), shape_(shape) {}

Type Meta::GetType() const { return type_; }

const std::vector<int64_t> &Meta::GetShape() const { return shape_; }

Meta Meta::AlignLeftTo(size_t size, float64_t value) const {
  std::vector<int64_t> shape(shape_);
  if (shape.size() < size) shape.insert(shape.begin(), size - shape.size(), static_cast<int64_t>(value));
  return Meta(type_, std::move(shape));
}

size_t Meta::GetElementsNum() const {
  size_t n = 1;
  for (int64_t dim : shape_) n *= static_cast<size_t>(dim);
  return n;
}

size_t Meta::GetSize() const { return GetElementsNum() * fluidml::GetSize(type_); }

size_t Meta::GetHashCode() const {
  size_t hash = std::hash<Type>()(type_);
  for (int64_t dim : shape_) Combine(hash, std::hash<int64_t>()(dim));
  return hash;
}

bool operator==(const Meta &lhs, const Meta &rhs) { return lhs.type_ == rhs.type_ && lhs.shape_ == rhs.shape_; }
bool operator!=(const Meta &lhs, const Meta &rhs) { return !(lhs == rhs); }

std::optional<Meta> BroadcastShape(const Meta &lhs, const Meta &rhs, Type type) {
  const size_t rank = std::max(lhs.GetShape().size(), rhs.GetShape().size());
  const Meta l = lhs.AlignLeftTo(rank), r = rhs.AlignLeftTo(rank);
  std::optional<std::vector<int64_t>> dims = BroadcastDims(l.GetShape(), r.GetShape(), rank);
  if (!dims) return std::nullopt;
  return Meta(type, std::move(*dims));
}

std::optional<Meta> BroadcastMatMulShape(const Meta &lhs, const Meta &rhs, Type type) {
  if (lhs.GetShape().size() < 2 || rhs.GetShape().size() < 2) return std::nullopt;
  const size_t rank = std::max(lhs.GetShape().size(), rhs.GetShape().size());
  const Meta l = lhs.AlignLeftTo(rank), r = rhs.AlignLeftTo(rank);
  const std::vector<int64_t> &ls = l.GetShape(), &rs = r.GetShape();
  if (rs[rank - 2] != ls[rank - 1]) return std::nullopt;
  std::optional<std::vector<int64_t>> dims = BroadcastDims(ls, rs, rank - 2);
  if (!dims) return std::nullopt;
  dims->push_back(ls[rank - 2]);
  dims->push_back(rs[rank - 1]);
  return Meta(type, std::move(*dims));
}

std::optional<Meta> ReshapeShapeInference(const Meta &shape, size_t items) {
  std::vector<int64_t> dims(shape.GetShape());
  int64_t wildcard = -1;
  size_t product = 1;
  for (size_t i = 0; i < dims.size(); ++i) {
    if (dims[i] == -1) {
      if (wildcard != -1) return std::nullopt;
      wildcard = static_cast<int64_t>(i);
    } else {
      product *= static_cast<size_t>(dims[i]);
    }
  }
  if (wildcard != -1) {
    if (items % product != 0) return std::nullopt;
    dims[wildcard] = static_cast<int64_t>(items / product);
  }
  return Meta(shape.GetType(), std::move(dims));
}

}  // namespace fluidml
