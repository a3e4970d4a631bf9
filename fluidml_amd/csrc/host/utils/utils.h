// Layout / order helpers of the data model (reference include/utils/utils.h,
// src/utils/utils.cpp:26-125).  A layout maps logical dim i to physical
// position layout[i]; strides are in elements.
#ifndef FLUIDML_AMD_HOST_UTILS_UTILS_H_
#define FLUIDML_AMD_HOST_UTILS_UTILS_H_

#include <cstddef>
#include <cstdint>
#include <vector>

namespace fluidml {
namespace utils {

// All permutations of 0..len-1 in the reference's enumeration order: order k
// of length n comes from order k/n of length n-1 with n-1 inserted at position
// k%n, so element 0 is the fully reversed permutation (utils.cpp:26-41). The
// layout DP breaks cost ties by this order.
std::vector<std::vector<size_t>> GenAllOrders(size_t len);
// Every index of `shape` in row-major order (utils.cpp:43-62).
std::vector<std::vector<size_t>> GenAllIndicesInOrder(const std::vector<int64_t> &shape);
// physical_shape[layout[i]] = shape[i] (utils.cpp:64-76).
std::vector<int64_t> GenPhysicalShape(const std::vector<int64_t> &shape, const std::vector<size_t> &layout);
// Row-major strides of `shape` (utils.cpp:78-83).
std::vector<int64_t> GenStrides(const std::vector<int64_t> &shape);
// strides[i] = rowmajor(physical_shape)[layout[i]] (utils.cpp:85-102).
std::vector<int64_t> GenStrides(const std::vector<int64_t> &shape, const std::vector<size_t> &layout);
std::vector<size_t> GenDefaultLayout(size_t rank);
std::vector<size_t> GenDefaultLayout(const std::vector<int64_t> &shape);
size_t GenIndex(const std::vector<size_t> &indices, const std::vector<int64_t> &strides);

}  // namespace utils
}  // namespace fluidml

#endif
