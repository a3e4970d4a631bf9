// ONNX-level graph (reference include/structure/graph/{graph,node,edge,attribute}.h).
// Values ("edges") and operators ("nodes") are kept by name in unordered maps
// exactly as the reference keeps them (graph.h:70-82): the order in which those
// maps iterate seeds the order of everything downstream (flow containers,
// topological order, lifetimes, heap ties), so the container types and the
// insertion calls are part of the memory plan's contract.
#ifndef FLUIDML_AMD_HOST_STRUCTURE_GRAPH_GRAPH_H_
#define FLUIDML_AMD_HOST_STRUCTURE_GRAPH_GRAPH_H_

#include <memory>
#include <optional>
#include <string>
#include <unordered_map>
#include <variant>
#include <vector>

#include "structure/tensor/meta.h"
#include "structure/tensor/tensor.h"

namespace fluidml {
namespace graph {

// Node attribute (reference attribute.h:14-48).
class Attribute {
 public:
  enum class Type { DataType, Int64, Float32, Int64Array, Tensor };
  explicit Attribute(fluidml::Type data) : value_(data) {}
  explicit Attribute(int64_t data) : value_(data) {}
  explicit Attribute(float32_t data) : value_(data) {}
  explicit Attribute(std::vector<int64_t> &&data) : value_(std::move(data)) {}
  explicit Attribute(Tensor &&data) : value_(std::move(data)) {}
  Type GetType() const { return static_cast<Type>(value_.index()); }
  fluidml::Type GetDataType() const { return std::get<fluidml::Type>(value_); }
  int64_t GetInt64() const { return std::get<int64_t>(value_); }
  float32_t GetFloat32() const { return std::get<float32_t>(value_); }
  const std::vector<int64_t> &GetInt64Array() const { return std::get<std::vector<int64_t>>(value_); }
  const Tensor &GetTensor() const { return std::get<Tensor>(value_); }

 private:
  std::variant<fluidml::Type, int64_t, float32_t, std::vector<int64_t>, Tensor> value_;
};

// A named value.  The reference models the five kinds as a class hierarchy
// (edge.h:14-108); one tagged class carries the same information.
class Edge {
 public:
  enum class Kind {
    ConstantScalar,  // rank-0 initializer (parser.cpp:226-237)
    ConstantTensor,  // initializer of rank >= 1
    Pure,            // graph.value_info
    Input,           // graph.input
    Output           // graph.output
  };
  static std::shared_ptr<Edge> MakeScalar(std::string &&name, Type type, float64_t value);
  static std::shared_ptr<Edge> MakeTensor(std::string &&name, Tensor &&tensor);
  static std::shared_ptr<Edge> MakeVariable(Kind kind, std::string &&name, Type type, std::vector<int64_t> &&shape);

  const std::string &GetName() const { return name_; }
  Kind GetKind() const { return kind_; }
  bool IsConstant() const { return kind_ == Kind::ConstantScalar || kind_ == Kind::ConstantTensor; }
  bool IsConstantScalar() const { return kind_ == Kind::ConstantScalar; }
  bool IsConstantTensor() const { return kind_ == Kind::ConstantTensor; }
  bool IsNonConstant() const { return !IsConstant(); }
  Type GetType() const { return meta_.GetType(); }
  const std::vector<int64_t> &GetShape() const { return meta_.GetShape(); }
  const Meta &GetMeta() const { return meta_; }
  float64_t GetScalar() const { return scalar_; }
  const Tensor &GetTensor() const { return *tensor_; }

 private:
  Edge(Kind kind, std::string &&name, Meta &&meta) : kind_(kind), name_(std::move(name)), meta_(std::move(meta)) {}
  Kind kind_;
  std::string name_;
  Meta meta_;
  float64_t scalar_ = 0;
  std::optional<Tensor> tensor_;
};

class Node {
 public:
  // the operator set the reference's parser accepts plus its three fused forms (node.h:17-56)
  enum class Op {
    Add, AddDivErfAddMulMul, AveragePool, Cast, Clip, Concat, ConstantOfShape, Conv, CumSum, Div, Dropout, Equal,
    Erf, Flatten, Gather, GatherAddAdd, Gemm, LayerNormalization, MatMul, MaxPool, Mul, Neg, Not, Pad, Pow,
    ReduceMean, Relu, Reshape, Slice, Softmax, Sqrt, Squeeze, Sub, Tanh, Transpose, Unsqueeze, UnsqueezeSubMul,
    Where,
  };
  Node(std::string &&name, Op op, std::unordered_map<std::string, Attribute> &&attributes = {})
      : name_(std::move(name)), op_(op), attributes_(std::move(attributes)) {}
  const std::string &GetName() const { return name_; }
  Op GetOp() const { return op_; }
  bool HasAttribute(const std::string &name) const { return attributes_.find(name) != attributes_.end(); }
  const Attribute &GetAttribute(const std::string &name) const { return attributes_.at(name); }
  const std::unordered_map<std::string, Attribute> &GetAttributes() const { return attributes_; }

 private:
  std::string name_;
  Op op_;
  std::unordered_map<std::string, Attribute> attributes_;
};

// ONNX op_type string -> Op; nullopt for operators the reference's parser does
// not know (parser.cpp:250-319).
std::optional<Node::Op> OpFromString(const std::string &op_type);
const char *OpToString(Node::Op op);

class Graph {
 public:
  Graph() = default;
  Graph(const Graph &) = delete;
  Graph(Graph &&) = default;
  Graph &operator=(Graph &&) = default;

  bool ExistEdge(const std::string &name) const;
  bool PutEdge(std::shared_ptr<Edge> &&edge);   // false (and no change) when the name exists
  std::shared_ptr<Edge> GetEdge(const std::string &name) const;
  std::shared_ptr<Node> GetEdgeFrom(const std::string &edge_name) const;             // producer or nullptr
  std::vector<std::shared_ptr<Node>> GetEdgeTo(const std::string &edge_name) const;  // consumers, link order
  bool ExistNode(const std::string &name) const;
  bool PutNode(std::shared_ptr<Node> &&node);
  std::shared_ptr<Node> GetNode(const std::string &name) const;
  std::vector<std::shared_ptr<Edge>> GetNodeFrom(const std::string &node_name) const;  // inputs, link order
  std::vector<std::shared_ptr<Edge>> GetNodeTo(const std::string &node_name) const;    // outputs, link order
  std::vector<std::shared_ptr<Edge>> GetAllEdges() const;  // container iteration order
  std::vector<std::shared_ptr<Node>> GetAllNodes() const;  // container iteration order
  // Links are silently refused when either end is unknown (graph.cpp:343-351, 357-365).
  bool EdgeToNode(const std::string &edge_name, const std::string &node_name);
  bool NodeToEdge(const std::string &node_name, const std::string &edge_name);
  // Remove a node / a value together with every link that mentions it (what the reference's
  // Node::Delete / Edge::Delete do for the fusion passes, node.cpp and edge.cpp of structure/graph).
  void DeleteNode(const std::string &name);
  void DeleteEdge(const std::string &name);

 private:
  struct EdgeContainer {
    std::shared_ptr<Edge> ptr;
    std::optional<std::string> from;
    std::vector<std::string> to;
  };
  struct NodeContainer {
    std::shared_ptr<Node> ptr;
    std::vector<std::string> from;
    std::vector<std::string> to;
  };
  std::unordered_map<std::string, EdgeContainer> edges_;
  std::unordered_map<std::string, NodeContainer> nodes_;
};

}  // namespace graph
}  // namespace fluidml

#endif
