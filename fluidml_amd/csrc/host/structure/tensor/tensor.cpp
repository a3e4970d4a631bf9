#include "structure/tensor/tensor.h"

#include <cstring>
#include <functional>
#include <stdexcept>

#include "utils/utils.h"

namespace fluidml {

Tensor::Tensor(Meta &&meta)
    : meta_(std::move(meta)), data_(std::make_shared<std::vector<float64_t>>(meta_.GetElementsNum())) {}

Tensor::Tensor(Meta &&meta, std::vector<float64_t> &&data)
    : meta_(std::move(meta)), data_(std::make_shared<std::vector<float64_t>>(std::move(data))) {
  if (data_->size() != meta_.GetElementsNum()) throw std::invalid_argument("Tensor: value count != shape product");
}

Tensor::Tensor(Type type, std::vector<int64_t> &&shape) : Tensor(Meta(type, std::move(shape))) {}

Tensor::Tensor(Type type, std::vector<int64_t> &&shape, std::vector<float64_t> &&data)
    : Tensor(Meta(type, std::move(shape)), std::move(data)) {}

const std::vector<float64_t> &Tensor::Get() const { return *data_; }

size_t Tensor::Linear(const std::vector<size_t> &indices) const {
  const std::vector<int64_t> &shape = meta_.GetShape();
  size_t index = 0;
  for (size_t i = 0; i < indices.size(); ++i) {
    if (indices[i] >= static_cast<size_t>(shape[i])) throw std::out_of_range("Tensor::Get: index out of range");
    index = index * static_cast<size_t>(shape[i]) + indices[i];
  }
  return index;
}

float64_t &Tensor::Get(const std::vector<size_t> &indices) {
  if (data_.use_count() > 1) data_ = std::make_shared<std::vector<float64_t>>(*data_);
  return (*data_)[Linear(indices)];
}

const float64_t &Tensor::Get(const std::vector<size_t> &indices) const { return (*data_)[Linear(indices)]; }

const Meta &Tensor::GetMeta() const { return meta_; }
Type Tensor::GetType() const { return meta_.GetType(); }
const std::vector<int64_t> &Tensor::GetShape() const { return meta_.GetShape(); }

size_t Tensor::GetHashCode() const {
  size_t hash = meta_.GetHashCode();
  std::hash<float64_t> h;
  for (float64_t v : *data_) hash ^= h(v) + 0 + (hash << 6) + (hash >> 2);
  return hash;
}

bool operator==(const Tensor &lhs, const Tensor &rhs) {
  return lhs.meta_ == rhs.meta_ && (lhs.data_ == rhs.data_ || *lhs.data_ == *rhs.data_);
}
bool operator!=(const Tensor &lhs, const Tensor &rhs) { return !(lhs == rhs); }

namespace {
template <typename T>
void PackAs(const std::vector<float64_t> &values, const std::vector<int64_t> &shape,
            const std::vector<int64_t> &strides, bool gathered, uint8_t *dst) {
  T *out = reinterpret_cast<T *>(dst);
  const size_t rank = shape.size();
  std::vector<int64_t> index(rank, 0);
  int64_t offset = 0;
  for (size_t n = 0; n < values.size(); ++n) {
    if (gathered) {
      out[n] = static_cast<T>(values[static_cast<size_t>(offset)]);
    } else {
      out[offset] = static_cast<T>(values[n]);
    }
    for (size_t d = rank; d-- > 0;) {
      offset += strides[d];
      if (++index[d] < shape[d]) break;
      offset -= strides[d] * shape[d];
      index[d] = 0;
    }
  }
}
}  // namespace

std::vector<uint8_t> Tensor::Pack(const std::vector<size_t> &layout, bool gathered) const {
  const std::vector<int64_t> &shape = meta_.GetShape();
  const std::vector<int64_t> strides = utils::GenStrides(shape, layout);
  std::vector<uint8_t> bytes(meta_.GetSize());
  switch (meta_.GetType()) {
    case Type::kBool: PackAs<uint8_t>(*data_, shape, strides, gathered, bytes.data()); break;
    case Type::kInt32: PackAs<int32_t>(*data_, shape, strides, gathered, bytes.data()); break;
    case Type::kInt64: PackAs<int64_t>(*data_, shape, strides, gathered, bytes.data()); break;
    case Type::kFloat32: PackAs<float32_t>(*data_, shape, strides, gathered, bytes.data()); break;
    case Type::kFloat64: PackAs<float64_t>(*data_, shape, strides, gathered, bytes.data()); break;
    default: throw std::invalid_argument("Tensor::Pack: unsupported element type");
  }
  return bytes;
}

}  // namespace fluidml
