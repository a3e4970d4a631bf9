#include "structure/flow/flow.h"

#include <stdexcept>

#include "utils/utils.h"

namespace fluidml {
namespace flow {

Region::Region(Kind kind, std::string &&name, Meta &&meta)
    : kind_(kind), name_(std::move(name)), meta_(std::move(meta)), layout_(utils::GenDefaultLayout(meta_.GetShape())) {}

Region::Region(Kind kind, std::string &&name, Meta &&meta, std::vector<size_t> &&layout)
    : kind_(kind), name_(std::move(name)), meta_(std::move(meta)), layout_(std::move(layout)) {}

Region::Region(std::string &&name, Tensor &&tensor)
    : kind_(Kind::Constant), name_(std::move(name)), meta_(tensor.GetMeta()),
      layout_(utils::GenDefaultLayout(meta_.GetShape())), tensor_(std::move(tensor)) {}

Region::Region(std::string &&name, Tensor &&tensor, std::vector<size_t> &&layout)
    : kind_(Kind::Constant), name_(std::move(name)), meta_(tensor.GetMeta()), layout_(std::move(layout)),
      tensor_(std::move(tensor)) {}

std::vector<int64_t> Region::GetPhysicalShape() const { return utils::GenPhysicalShape(meta_.GetShape(), layout_); }
std::vector<int64_t> Region::GetStrides() const { return utils::GenStrides(meta_.GetShape(), layout_); }

const Tensor &Region::GetTensor() const {
  if (!tensor_) throw std::logic_error("Region::GetTensor: " + name_ + " is not a constant region");
  return *tensor_;
}

const char *OpKindName(OpKind kind) {
  static const char *const kNames[] = {
      "AddConstant", "AddCommon", "AddDivErfAddMulMul", "AveragePoolWithoutPadding", "Cast", "Clip", "Concat2",
      "ConvWithoutPadding", "ConvWithPadding", "CumSum", "DivConstantRhs", "DivCommon", "Dropout", "Equal", "Erf",
      "Flatten", "GatherConstantIndexScalar", "GatherConstantIndicesTensor", "GatherConstantDataTensor",
      "GatherConstantDataTensorAddTensorLhsAddTensorLhs", "GemmConstantWeightsBias",
      "LayerNormalizationConstantScaleBias", "MatMul", "MaxPoolWithoutPadding", "MulConstant", "MulCommon", "Neg",
      "Not", "Pad", "Pow", "ReduceMean", "Relu", "Reshape", "Slice", "Softmax", "Sqrt", "Squeeze", "SubConstantLhs",
      "SubCommon", "Tanh", "Transpose", "Unsqueeze", "UnsqueezeSubLhsScalarMulRhsScalar",
      "WhereConstantCondConstantScalarY", "WhereConstantCondConstantTensorY"};
  return kNames[static_cast<size_t>(kind)];
}

Node::Node(std::string &&name, OpKind kind, std::shared_ptr<Region> &&input, std::shared_ptr<Region> &&output,
           Attrs &&attrs)
    : name_(std::move(name)), kind_(kind), lhs_(std::move(input)), rhs_(nullptr), output_(std::move(output)),
      attrs_(std::move(attrs)) {
  if (!lhs_ || !output_) throw std::invalid_argument("flow::Node " + name_ + ": null region");
}

Node::Node(std::string &&name, OpKind kind, std::shared_ptr<Region> &&lhs, std::shared_ptr<Region> &&rhs,
           std::shared_ptr<Region> &&output, Attrs &&attrs)
    : name_(std::move(name)), kind_(kind), lhs_(std::move(lhs)), rhs_(std::move(rhs)), output_(std::move(output)),
      attrs_(std::move(attrs)) {
  if (!lhs_ || !rhs_ || !output_) throw std::invalid_argument("flow::Node " + name_ + ": null region");
}

std::shared_ptr<Node> Node::Clone() const { return std::make_shared<Node>(*this); }

bool Node::HasBuffer() const {
  return kind_ == OpKind::Softmax || kind_ == OpKind::LayerNormalizationConstantScaleBias ||
         kind_ == OpKind::ConvWithPadding;
}

int64_t Node::GetAxis() const {
  const int64_t rank = static_cast<int64_t>(lhs_->GetMeta().GetShape().size());
  return attrs_.axis >= 0 ? attrs_.axis : rank + attrs_.axis;
}

size_t Node::GetBufferSize() const {
  switch (kind_) {
    case OpKind::Softmax:
    case OpKind::LayerNormalizationConstantScaleBias: {
      const Meta &meta = lhs_->GetMeta();
      std::vector<int64_t> shape = meta.GetShape();
      shape.at(static_cast<size_t>(GetAxis())) = 1;
      return Meta(meta.GetType(), std::move(shape)).GetSize();
    }
    case OpKind::ConvWithPadding: {
      const Meta &meta = lhs_->GetMeta();
      std::vector<int64_t> shape = meta.GetShape();
      const size_t spatial = shape.size() - 2;
      if (attrs_.pads.size() != 2 * spatial) throw std::logic_error("ConvWithPadding " + name_ + ": pads rank");
      for (size_t i = 0; i < spatial; ++i) shape[i + 2] += attrs_.pads[i] + attrs_.pads[i + spatial];
      return Meta(meta.GetType(), std::move(shape)).GetSize();
    }
    default: return 0;
  }
}

Edge::Edge(Kind kind, std::shared_ptr<Region> &&region, std::shared_ptr<Node> &&from, std::shared_ptr<Node> &&to)
    : kind_(kind), region_(std::move(region)), from_(std::move(from)), to_(std::move(to)) {
  if (!region_) throw std::invalid_argument("flow::Edge: null region");
  if (OwnsFrom() != (from_ != nullptr) || OwnsTo() != (to_ != nullptr)) {
    throw std::invalid_argument("flow::Edge " + region_->GetName() + ": ends do not match the edge kind");
  }
}

void Flow::PutNode(std::shared_ptr<Node> &&node) {
  std::string name = node->GetName();
  nodes_.insert({std::move(name), std::move(node)});
}

void Flow::PutEdge(std::shared_ptr<Edge> &&edge) {
  std::string name = edge->GetName();
  edges_.insert({std::move(name), std::move(edge)});
}

void Flow::PutRegion(std::shared_ptr<Region> &&region) {
  std::string name = region->GetName();
  regions_.insert({std::move(name), std::move(region)});
}

std::shared_ptr<Node> Flow::GetNode(const std::string &name) const {
  auto it = nodes_.find(name);
  return it == nodes_.end() ? nullptr : it->second;
}

std::shared_ptr<Region> Flow::GetRegion(const std::string &name) const {
  auto it = regions_.find(name);
  return it == regions_.end() ? nullptr : it->second;
}

std::vector<std::shared_ptr<Node>> Flow::GetNodes() const {
  std::vector<std::shared_ptr<Node>> out;
  for (const auto &kv : nodes_) out.push_back(kv.second);
  return out;
}

std::vector<std::shared_ptr<Edge>> Flow::GetEdges(const std::string &name) const {
  std::vector<std::shared_ptr<Edge>> out;
  auto range = edges_.equal_range(name);
  for (auto it = range.first; it != range.second; ++it) out.push_back(it->second);
  return out;
}

std::vector<std::shared_ptr<Edge>> Flow::GetEdges() const {
  std::vector<std::shared_ptr<Edge>> out;
  for (const auto &kv : edges_) out.push_back(kv.second);
  return out;
}

std::vector<std::shared_ptr<Region>> Flow::GetRegions() const {
  std::vector<std::shared_ptr<Region>> out;
  for (const auto &kv : regions_) out.push_back(kv.second);
  return out;
}

std::shared_ptr<Edge> Flow::FindTo(const std::string &region_name, const Node &node) const {
  auto range = edges_.equal_range(region_name);
  for (auto it = range.first; it != range.second; ++it) {
    if (it->second->OwnsTo() && it->second->GetTo().get() == &node) return it->second;
  }
  return nullptr;
}

std::shared_ptr<Edge> Flow::GetInputEdge(const Node &node) const { return FindTo(node.GetInputAsString(), node); }
std::shared_ptr<Edge> Flow::GetLhsEdge(const Node &node) const { return FindTo(node.GetLhsAsString(), node); }
std::shared_ptr<Edge> Flow::GetRhsEdge(const Node &node) const { return FindTo(node.GetRhsAsString(), node); }

std::shared_ptr<Edge> Flow::GetOutputEdge(const Node &node) const {
  auto range = edges_.equal_range(node.GetOutputAsString());
  for (auto it = range.first; it != range.second; ++it) {
    if (it->second->OwnsFrom() && it->second->GetFrom().get() == &node) return it->second;
  }
  return nullptr;
}

bool Flow::Check() const {
  for (const auto &kv : nodes_) {
    const Node &node = *kv.second;
    if (!GetLhsEdge(node) || !GetOutputEdge(node)) return false;
    if (node.IsDoubleInputs() && !GetRhsEdge(node)) return false;
  }
  for (const auto &kv : edges_) {
    const Edge &edge = *kv.second;
    if (edge.OwnsFrom() && GetNode(edge.GetFrom()->GetName()) == nullptr) return false;
    if (edge.OwnsTo() && GetNode(edge.GetTo()->GetName()) == nullptr) return false;
  }
  return true;
}

bool Flow::IsNoOverlapFlow() const {
  for (const auto &kv : edges_) {
    if (!kv.second->IsMemory()) continue;
    size_t memory_edges = 0;
    auto range = edges_.equal_range(kv.first);
    for (auto it = range.first; it != range.second; ++it) memory_edges += it->second->IsMemory() ? 1 : 0;
    if (memory_edges != 1) return false;
  }
  return true;
}

size_t Sequence::GetIndex(const std::string &name) const {
  for (size_t i = 0; i < nodes_.size(); ++i) {
    if (nodes_[i]->GetName() == name) return i;
  }
  throw std::out_of_range("Sequence::GetIndex: unknown node " + name);
}

}  // namespace flow
}  // namespace fluidml
