#include "utils/type.h"

#include <stdexcept>

namespace fluidml {

Type GetType(std::int32_t onnx_type) {
  switch (onnx_type) {
    case 1: return Type::kFloat32;
    case 6: return Type::kInt32;
    case 7: return Type::kInt64;
    case 9: return Type::kBool;
    case 10: return Type::kFloat16;
    default: return Type::kUnknown;
  }
}

size_t GetSize(Type type) {
  switch (type) {
    case Type::kBool: return sizeof(bool);
    case Type::kInt32: return sizeof(int32_t);
    case Type::kInt64: return sizeof(int64_t);
    case Type::kFloat32: return sizeof(float32_t);
    case Type::kFloat64: return sizeof(float64_t);
    default: throw std::invalid_argument("GetSize: element type has no size in FluidML");
  }
}

const char *GetStringFromType(Type type) {
  switch (type) {
    case Type::kBool: return "bool";
    case Type::kInt32: return "int32";
    case Type::kInt64: return "int64";
    case Type::kFloat32: return "float32";
    case Type::kFloat64: return "float64";
    default: throw std::invalid_argument("GetStringFromType: unnamed element type");
  }
}

}  // namespace fluidml
