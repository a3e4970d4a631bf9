#include "worker/converter.h"

#include <algorithm>
#include <cmath>
#include <stdexcept>

namespace fluidml {
namespace worker {
namespace {

using flow::Attrs;
using flow::OpKind;
using EdgePtr = std::shared_ptr<graph::Edge>;

[[noreturn]] void Unsupported(const graph::Node &node, const std::string &why) {
  throw std::runtime_error(std::string("converter: ") + graph::OpToString(node.GetOp()) + " node '" + node.GetName() +
                           "': " + why);
}

std::vector<int64_t> TensorAsInt64(const Tensor &t) {
  const std::vector<float64_t> &v = t.Get();
  std::vector<int64_t> out(v.size());
  for (size_t i = 0; i < v.size(); ++i) out[i] = static_cast<int64_t>(v[i]);
  return out;
}

struct Ctx {
  flow::Flow &flow;
  const graph::Graph &graph;
  const graph::Node &node;
  std::vector<EdgePtr> in, out;

  Ctx(flow::Flow &f, const graph::Graph &g, const graph::Node &n)
      : flow(f), graph(g), node(n), in(g.GetNodeFrom(n.GetName())), out(g.GetNodeTo(n.GetName())) {
    if (out.size() < 1) Unsupported(n, "no output with a declared shape (graph.output / value_info)");
    if (!out[0]->IsNonConstant()) Unsupported(n, "output is an initializer");
  }
  void Need(size_t n_inputs) const {
    if (in.size() != n_inputs) {
      Unsupported(node, "expects " + std::to_string(n_inputs) + " known inputs, has " + std::to_string(in.size()));
    }
  }
  std::shared_ptr<flow::Region> Region(const EdgePtr &edge) const {
    std::shared_ptr<flow::Region> r = flow.GetRegion(edge->GetName());
    if (!r) Unsupported(node, "no region for value '" + edge->GetName() + "'");
    return r;
  }
  std::string Name() const { return node.GetName(); }
  void PutSingle(OpKind kind, const EdgePtr &input, Attrs &&attrs = {}) const {
    flow.PutNode(std::make_shared<flow::Node>(Name(), kind, Region(input), Region(out[0]), std::move(attrs)));
  }
  void PutDouble(OpKind kind, const EdgePtr &lhs, const EdgePtr &rhs, Attrs &&attrs = {}) const {
    flow.PutNode(std::make_shared<flow::Node>(Name(), kind, Region(lhs), Region(rhs), Region(out[0]), std::move(attrs)));
  }
  int64_t Int(const char *key, int64_t fallback) const {
    return node.HasAttribute(key) ? node.GetAttribute(key).GetInt64() : fallback;
  }
  float64_t Float(const char *key, float64_t fallback) const {
    return node.HasAttribute(key) ? node.GetAttribute(key).GetFloat32() : fallback;
  }
  std::vector<int64_t> Ints(const char *key) const {
    if (!node.HasAttribute(key)) Unsupported(node, std::string("attribute '") + key + "' is required");
    return node.GetAttribute(key).GetInt64Array();
  }
};

// (NC,NC) | (NC,CT) | (CT,NC) -> Common; (NC,CS) | (CS,NC) -> Constant
// (reference converter.cpp:385-450 Add, 1608-1669 Mul)
void ConvertCommutative(const Ctx &c, OpKind common, OpKind constant) {
  c.Need(2);
  const EdgePtr &l = c.in[0], &r = c.in[1];
  if ((l->IsNonConstant() && r->IsNonConstant()) || (l->IsConstantTensor() && r->IsNonConstant()) ||
      (l->IsNonConstant() && r->IsConstantTensor())) {
    c.PutDouble(common, l, r);
  } else if ((l->IsNonConstant() && r->IsConstantScalar()) || (l->IsConstantScalar() && r->IsNonConstant())) {
    const EdgePtr &x = l->IsNonConstant() ? l : r, &k = l->IsNonConstant() ? r : l;
    Attrs a;
    a.type = k->GetType();
    a.value = k->GetScalar();
    c.PutSingle(constant, x, std::move(a));
  } else {
    Unsupported(c.node, "operand pattern not handled by FluidML");
  }
}

void ConvertUnary(const Ctx &c, OpKind kind) {
  c.Need(1);
  if (!c.in[0]->IsNonConstant()) Unsupported(c.node, "input is an initializer");
  c.PutSingle(kind, c.in[0]);
}

// `axes` as the second input (constant int64 tensor) or as an attribute
std::vector<int64_t> AxesOf(const Ctx &c) {
  if (c.in.size() == 2) {
    if (!c.in[1]->IsConstantTensor()) Unsupported(c.node, "axes must be a constant tensor");
    return TensorAsInt64(c.in[1]->GetTensor());
  }
  if (c.in.size() == 1) return c.Ints("axes");
  Unsupported(c.node, "expects 1 or 2 inputs");
}

void ConvertNode(flow::Flow &flow, const graph::Graph &graph, const graph::Node &node) {
  using Op = graph::Node::Op;
  const Ctx c(flow, graph, node);
  switch (node.GetOp()) {
    case Op::Add: ConvertCommutative(c, OpKind::AddCommon, OpKind::AddConstant); break;
    case Op::Mul: ConvertCommutative(c, OpKind::MulCommon, OpKind::MulConstant); break;
    case Op::Sub: {  // (CS,NC) -> c - x; (NC,NC) -> Common (converter.cpp:2284-2344)
      c.Need(2);
      if (c.in[0]->IsConstantScalar() && c.in[1]->IsNonConstant()) {
        Attrs a;
        a.type = c.in[0]->GetType();
        a.value = c.in[0]->GetScalar();
        c.PutSingle(OpKind::SubConstantLhs, c.in[1], std::move(a));
      } else if (c.in[0]->IsNonConstant() && c.in[1]->IsNonConstant()) {
        c.PutDouble(OpKind::SubCommon, c.in[0], c.in[1]);
      } else {
        Unsupported(node, "only (scalar - x) and (x - y) are handled by FluidML");
      }
      break;
    }
    case Op::Div: {  // (NC,CS) -> x / c; (NC,NC) -> Common (converter.cpp:941-993)
      c.Need(2);
      if (c.in[0]->IsNonConstant() && c.in[1]->IsConstantScalar()) {
        Attrs a;
        a.type = c.in[1]->GetType();
        a.value = c.in[1]->GetScalar();
        c.PutSingle(OpKind::DivConstantRhs, c.in[0], std::move(a));
      } else if (c.in[0]->IsNonConstant() && c.in[1]->IsNonConstant()) {
        c.PutDouble(OpKind::DivCommon, c.in[0], c.in[1]);
      } else {
        Unsupported(node, "only (x / scalar) and (x / y) are handled by FluidML");
      }
      break;
    }
    case Op::Pow: {  // (NC,CS) only (converter.cpp:1835-1854)
      c.Need(2);
      if (!c.in[0]->IsNonConstant() || !c.in[1]->IsConstantScalar()) Unsupported(node, "exponent must be a scalar initializer");
      Attrs a;
      a.type = c.in[1]->GetType();
      a.value = c.in[1]->GetScalar();
      c.PutSingle(OpKind::Pow, c.in[0], std::move(a));
      break;
    }
    case Op::Erf: ConvertUnary(c, OpKind::Erf); break;
    case Op::Relu: ConvertUnary(c, OpKind::Relu); break;
    case Op::Tanh: ConvertUnary(c, OpKind::Tanh); break;
    case Op::Sqrt: ConvertUnary(c, OpKind::Sqrt); break;
    case Op::Neg: ConvertUnary(c, OpKind::Neg); break;
    case Op::Not: ConvertUnary(c, OpKind::Not); break;
    case Op::Cast: ConvertUnary(c, OpKind::Cast); break;  // target type = output region's (converter.cpp:596-638)
    case Op::Clip: {  // min/max as scalar inputs or attributes (converter.cpp:664-690)
      Attrs a;
      if (c.in.size() == 3) {
        if (!c.in[1]->IsConstantScalar() || !c.in[2]->IsConstantScalar()) Unsupported(node, "min/max must be scalar initializers");
        a.min = static_cast<float32_t>(c.in[1]->GetScalar());
        a.max = static_cast<float32_t>(c.in[2]->GetScalar());
      } else {
        c.Need(1);
        if (!node.HasAttribute("min") || !node.HasAttribute("max")) Unsupported(node, "min and max are required");
        a.min = node.GetAttribute("min").GetFloat32();
        a.max = node.GetAttribute("max").GetFloat32();
      }
      c.PutSingle(OpKind::Clip, c.in[0], std::move(a));
      break;
    }
    case Op::Dropout: {  // identity; ratio from input 1 or attribute (converter.cpp:1004-1026)
      Attrs a;
      if (c.in.size() == 2 && c.in[1]->IsConstantScalar()) a.ratio = c.in[1]->GetScalar();
      else if (c.in.size() == 1) a.ratio = c.Float("ratio", 0.5);
      else Unsupported(node, "expects 1 input, or 2 with a scalar ratio");
      c.PutSingle(OpKind::Dropout, c.in[0], std::move(a));
      break;
    }
    case Op::Equal: {  // x == scalar (converter.cpp:1070-1105)
      c.Need(2);
      if (!c.in[0]->IsNonConstant() || !c.in[1]->IsConstantScalar()) Unsupported(node, "rhs must be a scalar initializer");
      Attrs a;
      a.type = c.in[1]->GetType();
      a.value = c.in[1]->GetScalar();
      c.PutSingle(OpKind::Equal, c.in[0], std::move(a));
      break;
    }
    case Op::CumSum: {  // axis is a scalar input (converter.cpp:873-919)
      c.Need(2);
      if (!c.in[1]->IsConstantScalar()) Unsupported(node, "axis must be a scalar initializer");
      Attrs a;
      a.axis = static_cast<int64_t>(c.in[1]->GetScalar());
      a.exclusive = c.Int("exclusive", 0) != 0;
      a.reverse = c.Int("reverse", 0) != 0;
      c.PutSingle(OpKind::CumSum, c.in[0], std::move(a));
      break;
    }
    case Op::Flatten: {
      c.Need(1);
      Attrs a;
      a.axis = c.Int("axis", 1);
      c.PutSingle(OpKind::Flatten, c.in[0], std::move(a));
      break;
    }
    case Op::Transpose: {  // perm defaults to the reversed order (converter.cpp:2413-2438)
      c.Need(1);
      Attrs a;
      if (node.HasAttribute("perm")) {
        a.perm = node.GetAttribute("perm").GetInt64Array();
      } else {
        const int64_t rank = static_cast<int64_t>(c.in[0]->GetShape().size());
        for (int64_t i = rank - 1; i >= 0; --i) a.perm.push_back(i);
      }
      c.PutSingle(OpKind::Transpose, c.in[0], std::move(a));
      break;
    }
    case Op::Reshape: {  // target shape = the output's declared shape (converter.cpp:1966-2023)
      c.Need(2);
      if (!c.in[0]->IsNonConstant() || !c.in[1]->IsConstantTensor()) Unsupported(node, "shape must be a constant tensor");
      c.PutSingle(OpKind::Reshape, c.in[0]);
      break;
    }
    case Op::Squeeze: {
      Attrs a;
      a.axes = AxesOf(c);
      c.PutSingle(OpKind::Squeeze, c.in[0], std::move(a));
      break;
    }
    case Op::Unsqueeze: {  // axes as constant tensor input only (converter.cpp:2455-2493)
      c.Need(2);
      if (!c.in[1]->IsConstantTensor()) Unsupported(node, "axes must be a constant tensor");
      Attrs a;
      a.axes = TensorAsInt64(c.in[1]->GetTensor());
      c.PutSingle(OpKind::Unsqueeze, c.in[0], std::move(a));
      break;
    }
    case Op::Slice: {  // starts, ends, axes, steps all 1-d constant tensors (converter.cpp:2035-2108)
      c.Need(5);
      for (int i = 1; i < 5; ++i) {
        if (!c.in[i]->IsConstantTensor() || c.in[i]->GetShape().size() != 1) Unsupported(node, "starts/ends/axes/steps must be 1-d constant tensors");
      }
      Attrs a;
      a.starts = TensorAsInt64(c.in[1]->GetTensor());
      a.ends = TensorAsInt64(c.in[2]->GetTensor());
      a.axes = TensorAsInt64(c.in[3]->GetTensor());
      a.steps = TensorAsInt64(c.in[4]->GetTensor());
      c.PutSingle(OpKind::Slice, c.in[0], std::move(a));
      break;
    }
    case Op::Pad: {  // pads tensor: begins then ends (converter.cpp:1759-1809)
      c.Need(2);
      if (!c.in[1]->IsConstantTensor()) Unsupported(node, "pads must be a constant tensor");
      const std::vector<int64_t> p = TensorAsInt64(c.in[1]->GetTensor());
      Attrs a;
      for (size_t i = 0; i < p.size() / 2; ++i) a.pad_pairs.push_back({p[i], p[i + p.size() / 2]});
      c.PutSingle(OpKind::Pad, c.in[0], std::move(a));
      break;
    }
    case Op::Concat: {  // exactly two non-constant inputs (converter.cpp:712-756)
      c.Need(2);
      if (!node.HasAttribute("axis")) Unsupported(node, "axis is required");
      Attrs a;
      a.axis = node.GetAttribute("axis").GetInt64();
      c.PutDouble(OpKind::Concat2, c.in[0], c.in[1], std::move(a));
      break;
    }
    case Op::Gather: {  // converter.cpp:1212-1290
      c.Need(2);
      Attrs a;
      // the reference stores the attribute in a size_t; a negative axis only
      // survives because it is converted back to int64 (converter.cpp:1212-1215)
      a.axis = c.Int("axis", 0);
      if (c.in[0]->IsNonConstant() && c.in[1]->IsConstantScalar()) {
        a.index = std::lround(c.in[1]->GetScalar());
        c.PutSingle(OpKind::GatherConstantIndexScalar, c.in[0], std::move(a));
      } else if (c.in[0]->IsNonConstant() && c.in[1]->IsConstantTensor()) {
        a.t0 = c.in[1]->GetTensor();
        c.PutSingle(OpKind::GatherConstantIndicesTensor, c.in[0], std::move(a));
      } else if (c.in[0]->IsConstantTensor() && c.in[1]->IsNonConstant()) {
        a.t0 = c.in[0]->GetTensor();
        c.PutSingle(OpKind::GatherConstantDataTensor, c.in[1], std::move(a));
      } else {
        Unsupported(node, "operand pattern not handled by FluidML");
      }
      break;
    }
    case Op::Where: {  // cond CT, x NC, y CS | CT (converter.cpp:2586-2629)
      c.Need(3);
      if (!c.in[0]->IsConstantTensor() || !c.in[1]->IsNonConstant()) Unsupported(node, "condition must be a constant tensor and x a variable");
      Attrs a;
      a.t0 = c.in[0]->GetTensor();
      if (c.in[2]->IsConstantScalar()) {
        a.type = c.in[2]->GetType();
        a.value = c.in[2]->GetScalar();
        c.PutSingle(OpKind::WhereConstantCondConstantScalarY, c.in[1], std::move(a));
      } else if (c.in[2]->IsConstantTensor()) {
        a.t1 = c.in[2]->GetTensor();
        c.PutSingle(OpKind::WhereConstantCondConstantTensorY, c.in[1], std::move(a));
      } else {
        Unsupported(node, "y must be an initializer");
      }
      break;
    }
    case Op::Softmax: {
      c.Need(1);
      Attrs a;
      a.axis = c.Int("axis", -1);
      c.PutSingle(OpKind::Softmax, c.in[0], std::move(a));
      break;
    }
    case Op::LayerNormalization: {  // X NC, scale CT, bias CT; axis default 1 (converter.cpp:1434-1485, node.h:672)
      c.Need(3);
      if (!c.in[0]->IsNonConstant() || !c.in[1]->IsConstantTensor() || !c.in[2]->IsConstantTensor()) Unsupported(node, "scale and bias must be constant tensors");
      Attrs a;
      a.axis = c.Int("axis", 1);
      a.epsilon = c.Float("epsilon", 1e-5);
      a.t0 = c.in[1]->GetTensor();
      a.t1 = c.in[2]->GetTensor();
      c.PutSingle(OpKind::LayerNormalizationConstantScaleBias, c.in[0], std::move(a));
      break;
    }
    case Op::ReduceMean: {  // keepdims attribute is required (converter.cpp:1905)
      Attrs a;
      a.axes = AxesOf(c);
      if (!node.HasAttribute("keepdims")) Unsupported(node, "keepdims is required");
      a.keepdims = node.GetAttribute("keepdims").GetInt64() != 0;
      c.PutSingle(OpKind::ReduceMean, c.in[0], std::move(a));
      break;
    }
    case Op::MaxPool: {  // kernel_shape, pads, strides required; pads all zero (converter.cpp:1551-1581)
      c.Need(1);
      Attrs a;
      a.kernel_shape = c.Ints("kernel_shape");
      a.pads = c.Ints("pads");
      a.strides = c.Ints("strides");
      if (!std::all_of(a.pads.begin(), a.pads.end(), [](int64_t p) { return p == 0; })) Unsupported(node, "padded MaxPool is not handled by FluidML");
      c.PutSingle(OpKind::MaxPoolWithoutPadding, c.in[0], std::move(a));
      break;
    }
    case Op::AveragePool: {  // kernel_shape required; dilations 1, pads 0, strides 1 (converter.cpp:551-592)
      c.Need(1);
      Attrs a;
      a.kernel_shape = c.Ints("kernel_shape");
      const size_t n = a.kernel_shape.size();
      a.dilations = node.HasAttribute("dilations") ? node.GetAttribute("dilations").GetInt64Array() : std::vector<int64_t>(n, 1);
      a.pads = node.HasAttribute("pads") ? node.GetAttribute("pads").GetInt64Array() : std::vector<int64_t>(2 * n, 0);
      a.strides = node.HasAttribute("strides") ? node.GetAttribute("strides").GetInt64Array() : std::vector<int64_t>(n, 1);
      if (!std::all_of(a.pads.begin(), a.pads.end(), [](int64_t p) { return p == 0; })) Unsupported(node, "padded AveragePool is not handled by FluidML");
      c.PutSingle(OpKind::AveragePoolWithoutPadding, c.in[0], std::move(a));
      break;
    }
    case Op::MatMul: {  // any two regions, at least one variable (converter.cpp:1488-1525)
      c.Need(2);
      if (c.in[0]->IsConstantScalar() || c.in[1]->IsConstantScalar()) Unsupported(node, "scalar operand");
      c.PutDouble(OpKind::MatMul, c.in[0], c.in[1]);
      break;
    }
    case Op::Gemm: {  // A NC, B CT, C CT; alpha and beta default to 0 when absent (converter.cpp:1394-1403)
      c.Need(3);
      if (!c.in[0]->IsNonConstant() || !c.in[1]->IsConstantTensor() || !c.in[2]->IsConstantTensor()) Unsupported(node, "B and C must be constant tensors");
      Attrs a;
      a.alpha = c.Float("alpha", 0.0);
      a.beta = c.Float("beta", 0.0);
      a.trans_a = c.Int("transA", 0) != 0;
      a.trans_b = c.Int("transB", 0) != 0;
      a.t0 = c.in[2]->GetTensor();
      c.PutDouble(OpKind::GemmConstantWeightsBias, c.in[0], c.in[1], std::move(a));
      break;
    }
    case Op::Conv: {  // X NC, W CT, optional B CT; all four list attributes required (converter.cpp:758-861)
      if (c.in.size() != 2 && c.in.size() != 3) Unsupported(node, "expects 2 or 3 inputs");
      if (!c.in[0]->IsNonConstant() || !c.in[1]->IsConstantTensor()) Unsupported(node, "weights must be a constant tensor");
      Attrs a;
      if (c.in.size() == 3) {
        if (!c.in[2]->IsConstantTensor()) Unsupported(node, "bias must be a constant tensor");
        a.t0 = c.in[2]->GetTensor();
      }
      a.group = c.Int("group", 1);
      a.dilations = c.Ints("dilations");
      a.kernel_shape = c.Ints("kernel_shape");
      a.pads = c.Ints("pads");
      a.strides = c.Ints("strides");
      const bool padded = !std::all_of(a.pads.begin(), a.pads.end(), [](int64_t p) { return p == 0; });
      c.PutDouble(padded ? OpKind::ConvWithPadding : OpKind::ConvWithoutPadding, c.in[0], c.in[1], std::move(a));
      break;
    }
    // the fused forms only arise from the graph passes; inputs = the chain's constants, then its variable
    case Op::AddDivErfAddMulMul: {  // add0 CT, div CS, add1 CS, mul1 CS, x (converter.cpp:455-520)
      c.Need(5);
      if (!c.in[0]->IsConstantTensor() || !c.in[1]->IsConstantScalar() || !c.in[2]->IsConstantScalar() ||
          !c.in[3]->IsConstantScalar() || !c.in[4]->IsNonConstant()) Unsupported(node, "operand pattern");
      Attrs a;
      a.t0 = c.in[0]->GetTensor();
      a.alpha = c.in[1]->GetScalar();
      a.beta = c.in[2]->GetScalar();
      a.extra = c.in[3]->GetScalar();
      c.PutSingle(OpKind::AddDivErfAddMulMul, c.in[4], std::move(a));
      break;
    }
    case Op::GatherAddAdd: {  // table CT, add0 CT, add1 CT, indices (converter.cpp:1293-1356)
      c.Need(4);
      if (!c.in[0]->IsConstantTensor() || !c.in[1]->IsConstantTensor() || !c.in[2]->IsConstantTensor() ||
          !c.in[3]->IsNonConstant()) Unsupported(node, "operand pattern");
      Attrs a;
      a.t0 = c.in[0]->GetTensor();
      a.t1 = c.in[1]->GetTensor();
      a.t2 = c.in[2]->GetTensor();
      c.PutSingle(OpKind::GatherConstantDataTensorAddTensorLhsAddTensorLhs, c.in[3], std::move(a));
      break;
    }
    case Op::UnsqueezeSubMul: {  // axes CT, sub CS, mul CS, x (converter.cpp:2496-2557)
      c.Need(4);
      if (!c.in[0]->IsConstantTensor() || !c.in[1]->IsConstantScalar() || !c.in[2]->IsConstantScalar() ||
          !c.in[3]->IsNonConstant()) Unsupported(node, "operand pattern");
      Attrs a;
      a.axes = TensorAsInt64(c.in[0]->GetTensor());
      a.alpha = c.in[1]->GetScalar();
      a.beta = c.in[2]->GetScalar();
      c.PutSingle(OpKind::UnsqueezeSubLhsScalarMulRhsScalar, c.in[3], std::move(a));
      break;
    }
    default:
      // ConstantOfShape is parsed but has no conversion (converter.cpp:268-274)
      Unsupported(node, "no flow node for this operator");
  }
}

class ConverterImpl : public Converter {
 public:
  flow::Flow Run(const graph::Graph &graph) override;
};

// Three sweeps in the graph's container order: regions for every value that
// has a shape, then one flow node per graph node, then def/use edges
// (reference converter.cpp:114-352).  Scalar initializers get neither a region
// nor an edge: they live inside the node that uses them.
flow::Flow ConverterImpl::Run(const graph::Graph &graph) {
  flow::Flow flow;
  for (const EdgePtr &edge : graph.GetAllEdges()) {
    std::string name = edge->GetName();
    switch (edge->GetKind()) {
      case graph::Edge::Kind::Input:
        flow.PutRegion(std::make_shared<flow::Region>(flow::Region::Kind::Input, std::move(name), Meta(edge->GetMeta())));
        break;
      case graph::Edge::Kind::Output:
        flow.PutRegion(std::make_shared<flow::Region>(flow::Region::Kind::Output, std::move(name), Meta(edge->GetMeta())));
        break;
      case graph::Edge::Kind::Pure:
        flow.PutRegion(std::make_shared<flow::Region>(flow::Region::Kind::Inner, std::move(name), Meta(edge->GetMeta())));
        break;
      case graph::Edge::Kind::ConstantTensor:
        flow.PutRegion(std::make_shared<flow::Region>(std::move(name), Tensor(edge->GetTensor())));
        break;
      case graph::Edge::Kind::ConstantScalar: break;
    }
  }
  for (const std::shared_ptr<graph::Node> &node : graph.GetAllNodes()) ConvertNode(flow, graph, *node);
  for (const EdgePtr &edge : graph.GetAllEdges()) {
    const std::string &name = edge->GetName();
    auto node_of = [&](const std::shared_ptr<graph::Node> &n) {
      std::shared_ptr<flow::Node> p = flow.GetNode(n->GetName());
      if (!p) throw std::runtime_error("converter: node '" + n->GetName() + "' was not converted");
      return p;
    };
    switch (edge->GetKind()) {
      case graph::Edge::Kind::Input:
        for (const auto &to : graph.GetEdgeTo(name)) {
          flow.PutEdge(std::make_shared<flow::Edge>(flow::Edge::Kind::Input, flow.GetRegion(name), nullptr, node_of(to)));
        }
        break;
      case graph::Edge::Kind::Output: {
        std::shared_ptr<graph::Node> from = graph.GetEdgeFrom(name);
        if (!from) throw std::runtime_error("converter: graph output '" + name + "' has no producer");
        flow.PutEdge(std::make_shared<flow::Edge>(flow::Edge::Kind::Output, flow.GetRegion(name), node_of(from), nullptr));
        for (const auto &to : graph.GetEdgeTo(name)) {  // an output that is also consumed inside the graph
          flow.PutEdge(std::make_shared<flow::Edge>(flow::Edge::Kind::Memory, flow.GetRegion(name), node_of(from), node_of(to)));
        }
        break;
      }
      case graph::Edge::Kind::Pure: {
        std::shared_ptr<graph::Node> from = graph.GetEdgeFrom(name);
        const auto tos = graph.GetEdgeTo(name);
        if (!from && !tos.empty()) throw std::runtime_error("converter: value '" + name + "' is used but never produced");
        for (const auto &to : tos) {
          flow.PutEdge(std::make_shared<flow::Edge>(flow::Edge::Kind::Memory, flow.GetRegion(name), node_of(from), node_of(to)));
        }
        break;
      }
      case graph::Edge::Kind::ConstantTensor:
        for (const auto &to : graph.GetEdgeTo(name)) {
          flow.PutEdge(std::make_shared<flow::Edge>(flow::Edge::Kind::Constant, flow.GetRegion(name), nullptr, node_of(to)));
        }
        break;
      case graph::Edge::Kind::ConstantScalar: break;
    }
  }
  if (!flow.Check()) throw std::runtime_error("converter: flow is not closed (a node lacks one of its edges)");
  return flow;
}

}  // namespace

std::unique_ptr<Converter> Converter::Make() { return std::make_unique<ConverterImpl>(); }

}  // namespace worker
}  // namespace fluidml
