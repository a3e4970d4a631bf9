// Element types of the FluidML data model (reference include/utils/type.h:11-29,
// src/utils/type.cpp:7-78).  The MLIR conversions of the reference have no
// counterpart here: the backend hands `static_cast<int>(Type)` to the C ABI,
// whose fl_dtype enum uses the same numbering.
#ifndef FLUIDML_AMD_HOST_UTILS_TYPE_H_
#define FLUIDML_AMD_HOST_UTILS_TYPE_H_

#include <cstddef>
#include <cstdint>

namespace fluidml {

using float32_t = float;
using float64_t = double;

enum class Type { kUnknown, kBool, kInt32, kInt64, kFloat16, kFloat32, kFloat64 };

// ONNX TensorProto.DataType -> Type (1 float, 6 int32, 7 int64, 9 bool, 10 float16).
Type GetType(std::int32_t onnx_type);
// Bytes per element; bool is one byte. Throws std::invalid_argument for
// kUnknown / kFloat16 (the reference leaves them unreachable).
size_t GetSize(Type type);
const char *GetStringFromType(Type type);

}  // namespace fluidml

#endif
