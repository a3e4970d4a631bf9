#include "utils/utils.h"

#include <numeric>
#include <stdexcept>

namespace fluidml {
namespace utils {

std::vector<std::vector<size_t>> GenAllOrders(size_t len) {
  std::vector<std::vector<size_t>> orders{{}};
  for (size_t n = 1; n <= len; ++n) {
    std::vector<std::vector<size_t>> grown;
    grown.reserve(orders.size() * n);
    for (const std::vector<size_t> &shorter : orders) {
      for (size_t pos = 0; pos < n; ++pos) {
        std::vector<size_t> order(shorter);
        order.insert(order.begin() + pos, n - 1);
        grown.push_back(std::move(order));
      }
    }
    orders.swap(grown);
  }
  return orders;
}

std::vector<std::vector<size_t>> GenAllIndicesInOrder(const std::vector<int64_t> &shape) {
  size_t total = 1;
  for (int64_t dim : shape) total *= static_cast<size_t>(dim);
  std::vector<std::vector<size_t>> indices;
  indices.reserve(total);
  std::vector<size_t> index(shape.size(), 0);
  for (size_t n = 0; n < total; ++n) {
    indices.push_back(index);
    for (size_t d = shape.size(); d-- > 0;) {
      if (++index[d] < static_cast<size_t>(shape[d])) break;
      index[d] = 0;
    }
  }
  return indices;
}

std::vector<int64_t> GenPhysicalShape(const std::vector<int64_t> &shape, const std::vector<size_t> &layout) {
  if (layout.size() != shape.size()) throw std::invalid_argument("GenPhysicalShape: layout rank != shape rank");
  std::vector<int64_t> physical(shape.size());
  for (size_t i = 0; i < shape.size(); ++i) {
    if (layout[i] >= shape.size()) throw std::invalid_argument("GenPhysicalShape: layout entry out of range");
    physical[layout[i]] = shape[i];
  }
  return physical;
}

std::vector<int64_t> GenStrides(const std::vector<int64_t> &shape) {
  std::vector<int64_t> strides(shape.size());
  int64_t running = 1;
  for (size_t i = shape.size(); i-- > 0;) {
    strides[i] = running;
    running *= shape[i];
  }
  return strides;
}

std::vector<int64_t> GenStrides(const std::vector<int64_t> &shape, const std::vector<size_t> &layout) {
  const std::vector<int64_t> physical_strides = GenStrides(GenPhysicalShape(shape, layout));
  std::vector<int64_t> strides(shape.size());
  for (size_t i = 0; i < shape.size(); ++i) strides[i] = physical_strides[layout[i]];
  return strides;
}

std::vector<size_t> GenDefaultLayout(size_t rank) {
  std::vector<size_t> layout(rank);
  std::iota(layout.begin(), layout.end(), size_t{0});
  return layout;
}

std::vector<size_t> GenDefaultLayout(const std::vector<int64_t> &shape) { return GenDefaultLayout(shape.size()); }

size_t GenIndex(const std::vector<size_t> &indices, const std::vector<int64_t> &strides) {
  size_t index = 0;
  for (size_t i = 0; i < indices.size(); ++i) index += indices[i] * static_cast<size_t>(strides[i]);
  return index;
}

}  // namespace utils
}  // namespace fluidml
