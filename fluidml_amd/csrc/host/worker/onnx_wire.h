// Dependency-free reader of the protobuf wire format for the slice of ONNX the
// FluidML parser consumes: ModelProto.graph with its nodes, initializers,
// inputs, outputs and value_info (reference src/worker/parser.cpp:193-332 reads
// exactly these through the generated onnx.pb.h, which is not available
// offline).  Field numbers are those of onnx/onnx.proto (IR version 3..10).
#ifndef FLUIDML_AMD_HOST_WORKER_ONNX_WIRE_H_
#define FLUIDML_AMD_HOST_WORKER_ONNX_WIRE_H_

#include <cstdint>
#include <optional>
#include <string>
#include <vector>

namespace fluidml {
namespace onnx_wire {

struct TensorData {
  std::string name;
  int32_t data_type = 0;  // TensorProto.DataType
  std::vector<int64_t> dims;
  bool has_raw_data = false;
  std::string raw_data;
  std::vector<float> float_data;
  std::vector<int32_t> int32_data;
  std::vector<int64_t> int64_data;
  std::vector<double> double_data;
};

struct AttributeData {
  enum Type { kUndefined = 0, kFloat = 1, kInt = 2, kString = 3, kTensor = 4, kGraph = 5, kFloats = 6, kInts = 7 };
  std::string name;
  int32_t type = kUndefined;
  float f = 0;
  int64_t i = 0;
  std::string s;
  std::vector<float> floats;
  std::vector<int64_t> ints;
  std::optional<TensorData> t;
};

struct NodeData {
  std::vector<std::string> input, output;
  std::string name, op_type;
  std::vector<AttributeData> attribute;
};

struct ValueInfoData {
  std::string name;
  int32_t elem_type = 0;
  bool has_shape = false;
  std::vector<int64_t> dims;  // dim_value of every dimension (0 for symbolic ones)
};

struct GraphData {
  std::string name;
  std::vector<NodeData> node;
  std::vector<TensorData> initializer;
  std::vector<ValueInfoData> input, output, value_info;
};

struct ModelData {
  int64_t ir_version = 0;
  GraphData graph;
};

// Throws std::runtime_error on truncated or malformed input.
ModelData ParseModel(const std::string &bytes);

}  // namespace onnx_wire
}  // namespace fluidml

#endif
