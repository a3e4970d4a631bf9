#include "worker/parser.h"

#include <cstring>
#include <fstream>
#include <iterator>
#include <stdexcept>

#include "worker/onnx_wire.h"

namespace fluidml {
namespace worker {
namespace {

using onnx_wire::AttributeData;
using onnx_wire::TensorData;

template <typename T>
std::vector<float64_t> RawAs(const std::string &raw) {
  std::vector<float64_t> data(raw.size() / sizeof(T));
  for (size_t i = 0; i < data.size(); ++i) {
    T v;
    std::memcpy(&v, raw.data() + i * sizeof(T), sizeof(T));
    data[i] = static_cast<float64_t>(v);
  }
  return data;
}

// Values of a TensorProto as float64: raw_data when present, else the typed
// repeated field that belongs to the element type (reference parser.cpp:44-84;
// bool and int32 share int32_data).
std::vector<float64_t> TensorValues(const TensorData &t, Type type) {
  switch (type) {
    case Type::kBool:
      if (t.has_raw_data) return RawAs<bool>(t.raw_data);
      return std::vector<float64_t>(t.int32_data.begin(), t.int32_data.end());
    case Type::kInt32:
      if (t.has_raw_data) return RawAs<int32_t>(t.raw_data);
      return std::vector<float64_t>(t.int32_data.begin(), t.int32_data.end());
    case Type::kInt64:
      if (t.has_raw_data) return RawAs<int64_t>(t.raw_data);
      return std::vector<float64_t>(t.int64_data.begin(), t.int64_data.end());
    case Type::kFloat32:
      if (t.has_raw_data) return RawAs<float32_t>(t.raw_data);
      return std::vector<float64_t>(t.float_data.begin(), t.float_data.end());
    case Type::kFloat64:
      if (t.has_raw_data) return RawAs<float64_t>(t.raw_data);
      return t.double_data;
    default:
      throw std::runtime_error("onnx tensor " + t.name + ": element type " + std::to_string(t.data_type) +
                               " is not handled by FluidML");
  }
}

Tensor MakeTensor(const TensorData &t) {
  const Type type = GetType(t.data_type);
  std::vector<int64_t> shape(t.dims);
  return Tensor(type, std::move(shape), TensorValues(t, type));
}

void CreateNode(graph::Graph &graph, const onnx_wire::NodeData &proto, graph::Node::Op op) {
  std::unordered_map<std::string, graph::Attribute> attributes;
  for (const AttributeData &a : proto.attribute) {
    std::string key = a.name;
    switch (a.type) {
      case AttributeData::kInt:
        // Cast's `to` is an element type (reference parser.cpp:93-99)
        if (op == graph::Node::Op::Cast) attributes.insert({std::move(key), graph::Attribute(GetType(static_cast<int32_t>(a.i)))});
        else attributes.insert({std::move(key), graph::Attribute(a.i)});
        break;
      case AttributeData::kFloat: attributes.insert({std::move(key), graph::Attribute(a.f)}); break;
      case AttributeData::kInts:
        attributes.insert({std::move(key), graph::Attribute(std::vector<int64_t>(a.ints))});
        break;
      case AttributeData::kTensor:
        if (!a.t) throw std::runtime_error("onnx node " + proto.name + ": TENSOR attribute without a tensor");
        attributes.insert({std::move(key), graph::Attribute(MakeTensor(*a.t))});
        break;
      default:
        throw std::runtime_error("onnx node " + proto.name + ": attribute " + a.name + " has a type FluidML does not read");
    }
  }
  std::string name = proto.name;
  graph.PutNode(std::make_shared<graph::Node>(std::move(name), op, std::move(attributes)));
  for (const std::string &input : proto.input) graph.EdgeToNode(input, proto.name);
  for (const std::string &output : proto.output) graph.NodeToEdge(proto.name, output);
}

void CreateVariable(graph::Graph &graph, graph::Edge::Kind kind, const onnx_wire::ValueInfoData &v) {
  std::string name = v.name;
  std::vector<int64_t> shape(v.dims);
  graph.PutEdge(graph::Edge::MakeVariable(kind, std::move(name), GetType(v.elem_type), std::move(shape)));
}

class ParserImpl : public Parser {
 public:
  graph::Graph RunOnBytes(const std::string &bytes) override;
};

// Insertion order is the file's: initializers, inputs, outputs, value_info,
// then nodes with their links (reference parser.cpp:199-249, 250-327).
graph::Graph ParserImpl::RunOnBytes(const std::string &bytes) {
  const onnx_wire::ModelData model = onnx_wire::ParseModel(bytes);
  graph::Graph graph;
  for (const TensorData &init : model.graph.initializer) {
    std::string name = init.name;
    const Type type = GetType(init.data_type);
    if (type != Type::kBool && type != Type::kInt32 && type != Type::kInt64 && type != Type::kFloat32) {
      throw std::runtime_error("onnx initializer " + init.name + ": element type not handled by FluidML");
    }
    if (!init.dims.empty()) {
      graph.PutEdge(graph::Edge::MakeTensor(std::move(name), MakeTensor(init)));
    } else {
      const std::vector<float64_t> values = TensorValues(init, type);
      if (values.size() != 1) throw std::runtime_error("onnx initializer " + init.name + ": rank 0 but not one value");
      graph.PutEdge(graph::Edge::MakeScalar(std::move(name), type, values[0]));
    }
  }
  for (const auto &v : model.graph.input) CreateVariable(graph, graph::Edge::Kind::Input, v);
  for (const auto &v : model.graph.output) CreateVariable(graph, graph::Edge::Kind::Output, v);
  for (const auto &v : model.graph.value_info) CreateVariable(graph, graph::Edge::Kind::Pure, v);
  for (const onnx_wire::NodeData &node : model.graph.node) {
    std::optional<graph::Node::Op> op = graph::OpFromString(node.op_type);
    if (!op || *op == graph::Node::Op::AddDivErfAddMulMul || *op == graph::Node::Op::GatherAddAdd ||
        *op == graph::Node::Op::UnsqueezeSubMul) {
      throw std::runtime_error("onnx node " + node.name + ": operator " + node.op_type + " is not supported by FluidML");
    }
    if (node.name.empty()) throw std::runtime_error("onnx: a " + node.op_type + " node has no name (names key the plan)");
    CreateNode(graph, node, *op);
  }
  return graph;
}

}  // namespace

std::unique_ptr<Parser> Parser::Make() { return std::make_unique<ParserImpl>(); }

graph::Graph Parser::Run(std::string_view path) {
  std::ifstream ifs(std::string(path), std::ios::binary);
  if (!ifs) throw std::runtime_error("cannot open " + std::string(path));
  return Run(ifs);
}

graph::Graph Parser::Run(std::istream &input) {
  std::string bytes((std::istreambuf_iterator<char>(input)), std::istreambuf_iterator<char>());
  return RunOnBytes(bytes);
}

}  // namespace worker
}  // namespace fluidml
