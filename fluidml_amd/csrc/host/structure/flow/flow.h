// Typed operator graph: the form in which the hot path is planned and launched
// (reference include/structure/flow/{region,node,edge,flow,sequence}.h).
//
// The reference spells every operator variant as its own C++ class (45 leaf
// classes over four virtual bases).  Here a node is plain data -- an OpKind, up
// to two input regions, one output region and an attribute record -- because
// on this backend nothing is generated per class: a node is looked up in a
// table and launched.  What planning depends on is kept exactly: node and
// region names, single/double input arity, scratch size per node
// (GetBufferSize), region kinds, edge kinds, and the unordered containers of
// Flow with their insertion order.
#ifndef FLUIDML_AMD_HOST_STRUCTURE_FLOW_FLOW_H_
#define FLUIDML_AMD_HOST_STRUCTURE_FLOW_FLOW_H_

#include <memory>
#include <optional>
#include <string>
#include <unordered_map>
#include <vector>

#include "structure/tensor/meta.h"
#include "structure/tensor/tensor.h"

namespace fluidml {
namespace flow {

// A tensor with a name and a layout (reference region.h:14-128).
class Region {
 public:
  enum class Kind { Inner, Input, Output, Constant };
  Region(Kind kind, std::string &&name, Meta &&meta);
  Region(Kind kind, std::string &&name, Meta &&meta, std::vector<size_t> &&layout);
  Region(std::string &&name, Tensor &&tensor);  // Constant
  Region(std::string &&name, Tensor &&tensor, std::vector<size_t> &&layout);
  Kind GetKind() const { return kind_; }
  const std::string &GetName() const { return name_; }
  const Meta &GetMeta() const { return meta_; }
  const std::vector<size_t> &GetLayout() const { return layout_; }
  std::vector<int64_t> GetPhysicalShape() const;
  std::vector<int64_t> GetStrides() const;
  void SetLayout(std::vector<size_t> &&layout) { layout_ = std::move(layout); }
  // only Inner regions live in the arena (region.cpp:57,66,94)
  bool NeedMemoryAllocation() const { return kind_ == Kind::Inner; }
  bool IsInterface() const { return kind_ == Kind::Input || kind_ == Kind::Output; }
  const Tensor &GetTensor() const;  // Constant only

 private:
  Kind kind_;
  std::string name_;
  Meta meta_;
  std::vector<size_t> layout_;
  std::optional<Tensor> tensor_;
};

// One value per reference kernel class; the spelling is the class name without
// the "Kernel"/"Node" suffix.
enum class OpKind {
  AddConstant, AddCommon, AddDivErfAddMulMul, AveragePoolWithoutPadding, Cast, Clip, Concat2,
  ConvWithoutPadding, ConvWithPadding, CumSum, DivConstantRhs, DivCommon, Dropout, Equal, Erf, Flatten,
  GatherConstantIndexScalar, GatherConstantIndicesTensor, GatherConstantDataTensor,
  GatherConstantDataTensorAddTensorLhsAddTensorLhs, GemmConstantWeightsBias, LayerNormalizationConstantScaleBias,
  MatMul, MaxPoolWithoutPadding, MulConstant, MulCommon, Neg, Not, Pad, Pow, ReduceMean, Relu, Reshape, Slice,
  Softmax, Sqrt, Squeeze, SubConstantLhs, SubCommon, Tanh, Transpose, Unsqueeze, UnsqueezeSubLhsScalarMulRhsScalar,
  WhereConstantCondConstantScalarY, WhereConstantCondConstantTensorY,
};
const char *OpKindName(OpKind kind);

// Attributes of all node variants in one record (reference node.h:139-1148).
// Unused fields keep their defaults; which are used is listed per kind in
// converter.cpp of this backend.
struct Attrs {
  Type type = Type::kUnknown;  // element type of `value` (Add/Div/Mul/Sub/Equal/Where constants)
  float64_t value = 0;         // scalar operand
  float64_t alpha = 0, beta = 0;  // Gemm; also div / add1 / mul1 of the fused GELU and sub / mul of the fused mask
  float64_t extra = 0;
  bool trans_a = false, trans_b = false;
  int64_t axis = 0;
  float64_t epsilon = 1e-5;
  int64_t group = 1;
  int64_t index = 0;
  float32_t min = 0, max = 0;
  bool keepdims = true, exclusive = false, reverse = false;
  float64_t ratio = 0.5;
  std::vector<int64_t> axes, dilations, kernel_shape, pads, strides, perm, starts, ends, steps;
  std::vector<std::tuple<int64_t, int64_t>> pad_pairs;  // Pad: (before, after) per dim
  // constants embedded in the node: Conv bias | Gemm bias | LN scale,bias |
  // Gather data / indices | fused-gather add weights | Where cond, y | GELU add0
  std::optional<Tensor> t0, t1, t2;
};

class Node {
 public:
  // single input
  Node(std::string &&name, OpKind kind, std::shared_ptr<Region> &&input, std::shared_ptr<Region> &&output,
       Attrs &&attrs = {});
  // double inputs
  Node(std::string &&name, OpKind kind, std::shared_ptr<Region> &&lhs, std::shared_ptr<Region> &&rhs,
       std::shared_ptr<Region> &&output, Attrs &&attrs = {});
  std::shared_ptr<Node> Clone() const;  // shares regions, copies attributes

  const std::string &GetName() const { return name_; }
  OpKind GetKind() const { return kind_; }
  const char *GetKindName() const { return OpKindName(kind_); }
  bool IsSingleInput() const { return rhs_ == nullptr; }
  bool IsDoubleInputs() const { return rhs_ != nullptr; }
  // which of the four kernel families serves this node (reference kernel.h:40-88)
  bool HasBuffer() const;
  // Scratch bytes the memory plan reserves under the node's name (reference
  // flow/node.cpp:500-519 padded conv input, :972-985 LayerNorm, :1355-1368 Softmax).
  size_t GetBufferSize() const;
  // axis normalised against the input rank (reference flow/node.cpp:931-933, 1370-1372)
  int64_t GetAxis() const;

  const std::shared_ptr<Region> &GetInput() const { return lhs_; }
  const std::shared_ptr<Region> &GetLhs() const { return lhs_; }
  const std::shared_ptr<Region> &GetRhs() const { return rhs_; }
  const std::shared_ptr<Region> &GetOutput() const { return output_; }
  const std::string &GetInputAsString() const { return lhs_->GetName(); }
  const std::string &GetLhsAsString() const { return lhs_->GetName(); }
  const std::string &GetRhsAsString() const { return rhs_->GetName(); }
  const std::string &GetOutputAsString() const { return output_->GetName(); }
  void SetInput(std::shared_ptr<Region> &&r) { lhs_ = std::move(r); }
  void SetLhs(std::shared_ptr<Region> &&r) { lhs_ = std::move(r); }
  void SetRhs(std::shared_ptr<Region> &&r) { rhs_ = std::move(r); }
  void SetOutput(std::shared_ptr<Region> &&r) { output_ = std::move(r); }
  const Attrs &GetAttrs() const { return attrs_; }

 private:
  std::string name_;
  OpKind kind_;
  std::shared_ptr<Region> lhs_, rhs_, output_;
  Attrs attrs_;
};

// def/use link between a region and nodes (reference edge.h:11-116).
class Edge {
 public:
  enum class Kind {
    Memory,    // node -> node through a region
    Input,     // graph input -> node
    Output,    // node -> graph output
    Constant   // constant region -> node
  };
  Edge(Kind kind, std::shared_ptr<Region> &&region, std::shared_ptr<Node> &&from, std::shared_ptr<Node> &&to);
  Kind GetKind() const { return kind_; }
  bool IsMemory() const { return kind_ == Kind::Memory; }
  bool OwnsFrom() const { return kind_ == Kind::Memory || kind_ == Kind::Output; }
  bool OwnsTo() const { return kind_ != Kind::Output; }
  const std::shared_ptr<Region> &GetRegion() const { return region_; }
  const std::string &GetName() const { return region_->GetName(); }
  const Meta &GetMeta() const { return region_->GetMeta(); }
  const std::vector<size_t> &GetLayout() const { return region_->GetLayout(); }
  const std::shared_ptr<Node> &GetFrom() const { return from_; }
  const std::shared_ptr<Node> &GetTo() const { return to_; }

 private:
  Kind kind_;
  std::shared_ptr<Region> region_;
  std::shared_ptr<Node> from_, to_;
};

class Flow {
 public:
  Flow() = default;
  Flow(const Flow &) = delete;
  Flow(Flow &&) = default;
  Flow &operator=(Flow &&) = default;
  void PutNode(std::shared_ptr<Node> &&node);
  void PutEdge(std::shared_ptr<Edge> &&edge);
  void PutRegion(std::shared_ptr<Region> &&region);
  std::shared_ptr<Node> GetNode(const std::string &name) const;
  std::shared_ptr<Region> GetRegion(const std::string &name) const;
  // all of these return container iteration order (reference flow.cpp:78-110)
  std::vector<std::shared_ptr<Node>> GetNodes() const;
  std::vector<std::shared_ptr<Edge>> GetEdges(const std::string &name) const;
  std::vector<std::shared_ptr<Edge>> GetEdges() const;
  std::vector<std::shared_ptr<Region>> GetRegions() const;
  // the edge named after the node's input/lhs/rhs region that ends at this node
  std::shared_ptr<Edge> GetInputEdge(const Node &node) const;
  std::shared_ptr<Edge> GetLhsEdge(const Node &node) const;
  std::shared_ptr<Edge> GetRhsEdge(const Node &node) const;
  std::shared_ptr<Edge> GetOutputEdge(const Node &node) const;
  // every node has its edges and every edge has its nodes (reference flow.cpp:192-295)
  bool Check() const;
  // every Memory edge's region name is used by exactly one Memory edge (reference flow.cpp:316-337)
  bool IsNoOverlapFlow() const;

 private:
  std::shared_ptr<Edge> FindTo(const std::string &region_name, const Node &node) const;
  std::unordered_map<std::string, std::shared_ptr<Node>> nodes_;
  std::unordered_multimap<std::string, std::shared_ptr<Edge>> edges_;
  std::unordered_map<std::string, std::shared_ptr<Region>> regions_;
};

// A flow with its nodes in execution order (reference sequence.h:12-31).
class Sequence {
 public:
  Sequence() = default;
  Sequence(const Sequence &) = delete;
  Sequence(Sequence &&) = default;
  Sequence &operator=(Sequence &&) = default;
  void PutNode(std::shared_ptr<Node> &&node) { nodes_.push_back(std::move(node)); }
  void PutEdge(std::shared_ptr<Edge> &&edge) { edges_.push_back(std::move(edge)); }
  void PutRegion(std::shared_ptr<Region> &&region) { regions_.push_back(std::move(region)); }
  size_t GetIndex(const std::string &name) const;  // throws std::out_of_range for an unknown node
  const std::vector<std::shared_ptr<Node>> &GetNodes() const { return nodes_; }
  const std::vector<std::shared_ptr<Edge>> &GetEdges() const { return edges_; }
  const std::vector<std::shared_ptr<Region>> &GetRegions() const { return regions_; }

 private:
  std::vector<std::shared_ptr<Node>> nodes_;
  std::vector<std::shared_ptr<Edge>> edges_;
  std::vector<std::shared_ptr<Region>> regions_;
};

}  // namespace flow
}  // namespace fluidml

#endif
