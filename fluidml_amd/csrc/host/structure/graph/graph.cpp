#include "structure/graph/graph.h"

#include <algorithm>

#include <stdexcept>
#include <utility>

namespace fluidml {
namespace graph {

std::shared_ptr<Edge> Edge::MakeScalar(std::string &&name, Type type, float64_t value) {
  std::shared_ptr<Edge> e(new Edge(Kind::ConstantScalar, std::move(name), Meta(type, std::vector<int64_t>{})));
  e->scalar_ = value;
  return e;
}

std::shared_ptr<Edge> Edge::MakeTensor(std::string &&name, Tensor &&tensor) {
  std::shared_ptr<Edge> e(new Edge(Kind::ConstantTensor, std::move(name), Meta(tensor.GetMeta())));
  e->tensor_ = std::move(tensor);
  return e;
}

std::shared_ptr<Edge> Edge::MakeVariable(Kind kind, std::string &&name, Type type, std::vector<int64_t> &&shape) {
  if (kind != Kind::Pure && kind != Kind::Input && kind != Kind::Output) {
    throw std::invalid_argument("Edge::MakeVariable: kind must be Pure, Input or Output");
  }
  return std::shared_ptr<Edge>(new Edge(kind, std::move(name), Meta(type, std::move(shape))));
}

namespace {
const std::pair<const char *, Node::Op> kOps[] = {
    {"Add", Node::Op::Add}, {"AveragePool", Node::Op::AveragePool}, {"Cast", Node::Op::Cast},
    {"Clip", Node::Op::Clip}, {"Concat", Node::Op::Concat}, {"ConstantOfShape", Node::Op::ConstantOfShape},
    {"Conv", Node::Op::Conv}, {"CumSum", Node::Op::CumSum}, {"Div", Node::Op::Div}, {"Dropout", Node::Op::Dropout},
    {"Equal", Node::Op::Equal}, {"Erf", Node::Op::Erf}, {"Flatten", Node::Op::Flatten}, {"Gather", Node::Op::Gather},
    {"Gemm", Node::Op::Gemm}, {"LayerNormalization", Node::Op::LayerNormalization}, {"MatMul", Node::Op::MatMul},
    {"MaxPool", Node::Op::MaxPool}, {"Mul", Node::Op::Mul}, {"Neg", Node::Op::Neg}, {"Not", Node::Op::Not},
    {"Pad", Node::Op::Pad}, {"Pow", Node::Op::Pow}, {"ReduceMean", Node::Op::ReduceMean}, {"Relu", Node::Op::Relu},
    {"Reshape", Node::Op::Reshape}, {"Slice", Node::Op::Slice}, {"Softmax", Node::Op::Softmax},
    {"Sqrt", Node::Op::Sqrt}, {"Squeeze", Node::Op::Squeeze}, {"Sub", Node::Op::Sub}, {"Tanh", Node::Op::Tanh},
    {"Transpose", Node::Op::Transpose}, {"Unsqueeze", Node::Op::Unsqueeze}, {"Where", Node::Op::Where},
    // fused forms produced by graph passes, never by ONNX files
    {"AddDivErfAddMulMul", Node::Op::AddDivErfAddMulMul}, {"GatherAddAdd", Node::Op::GatherAddAdd},
    {"UnsqueezeSubMul", Node::Op::UnsqueezeSubMul},
};
}  // namespace

std::optional<Node::Op> OpFromString(const std::string &op_type) {
  for (const auto &entry : kOps) {
    if (op_type == entry.first) return entry.second;
  }
  return std::nullopt;
}

const char *OpToString(Node::Op op) {
  for (const auto &entry : kOps) {
    if (entry.second == op) return entry.first;
  }
  return "?";
}

bool Graph::ExistEdge(const std::string &name) const { return edges_.find(name) != edges_.end(); }

bool Graph::PutEdge(std::shared_ptr<Edge> &&edge) {
  std::string name = edge->GetName();
  if (ExistEdge(name)) return false;
  edges_[name] = EdgeContainer{std::move(edge), {}, {}};
  return true;
}

std::shared_ptr<Edge> Graph::GetEdge(const std::string &name) const {
  auto it = edges_.find(name);
  return it == edges_.end() ? nullptr : it->second.ptr;
}

std::shared_ptr<Node> Graph::GetEdgeFrom(const std::string &edge_name) const {
  auto it = edges_.find(edge_name);
  if (it == edges_.end()) throw std::out_of_range("graph: unknown edge " + edge_name);
  if (!it->second.from) return nullptr;
  return GetNode(*it->second.from);
}

std::vector<std::shared_ptr<Node>> Graph::GetEdgeTo(const std::string &edge_name) const {
  auto it = edges_.find(edge_name);
  if (it == edges_.end()) throw std::out_of_range("graph: unknown edge " + edge_name);
  std::vector<std::shared_ptr<Node>> result;
  for (const std::string &name : it->second.to) {
    if (std::shared_ptr<Node> node = GetNode(name)) result.push_back(std::move(node));
  }
  return result;
}

bool Graph::ExistNode(const std::string &name) const { return nodes_.find(name) != nodes_.end(); }

bool Graph::PutNode(std::shared_ptr<Node> &&node) {
  std::string name = node->GetName();
  if (ExistNode(name)) return false;
  nodes_[name] = NodeContainer{std::move(node), {}, {}};
  return true;
}

std::shared_ptr<Node> Graph::GetNode(const std::string &name) const {
  auto it = nodes_.find(name);
  return it == nodes_.end() ? nullptr : it->second.ptr;
}

std::vector<std::shared_ptr<Edge>> Graph::GetNodeFrom(const std::string &node_name) const {
  auto it = nodes_.find(node_name);
  if (it == nodes_.end()) throw std::out_of_range("graph: unknown node " + node_name);
  std::vector<std::shared_ptr<Edge>> result;
  for (const std::string &name : it->second.from) {
    if (std::shared_ptr<Edge> edge = GetEdge(name)) result.push_back(std::move(edge));
  }
  return result;
}

std::vector<std::shared_ptr<Edge>> Graph::GetNodeTo(const std::string &node_name) const {
  auto it = nodes_.find(node_name);
  if (it == nodes_.end()) throw std::out_of_range("graph: unknown node " + node_name);
  std::vector<std::shared_ptr<Edge>> result;
  for (const std::string &name : it->second.to) {
    if (std::shared_ptr<Edge> edge = GetEdge(name)) result.push_back(std::move(edge));
  }
  return result;
}

std::vector<std::shared_ptr<Edge>> Graph::GetAllEdges() const {
  std::vector<std::shared_ptr<Edge>> result;
  for (const auto &entry : edges_) result.push_back(entry.second.ptr);
  return result;
}

std::vector<std::shared_ptr<Node>> Graph::GetAllNodes() const {
  std::vector<std::shared_ptr<Node>> result;
  for (const auto &entry : nodes_) result.push_back(entry.second.ptr);
  return result;
}

bool Graph::EdgeToNode(const std::string &edge_name, const std::string &node_name) {
  if (!ExistEdge(edge_name) || !ExistNode(node_name)) return false;
  edges_[edge_name].to.push_back(node_name);
  nodes_[node_name].from.push_back(edge_name);
  return true;
}

bool Graph::NodeToEdge(const std::string &node_name, const std::string &edge_name) {
  if (!ExistNode(node_name) || !ExistEdge(edge_name)) return false;
  nodes_[node_name].to.push_back(edge_name);
  edges_[edge_name].from = node_name;
  return true;
}

namespace {
void Scrub(std::vector<std::string> *names, const std::string &name) {
  names->erase(std::remove(names->begin(), names->end(), name), names->end());
}
}  // namespace

void Graph::DeleteNode(const std::string &name) {
  if (nodes_.erase(name) == 0) return;
  for (auto &kv : edges_) {
    if (kv.second.from && *kv.second.from == name) kv.second.from.reset();
    Scrub(&kv.second.to, name);
  }
}

void Graph::DeleteEdge(const std::string &name) {
  if (edges_.erase(name) == 0) return;
  for (auto &kv : nodes_) {
    Scrub(&kv.second.from, name);
    Scrub(&kv.second.to, name);
  }
}

}  // namespace graph
}  // namespace fluidml
