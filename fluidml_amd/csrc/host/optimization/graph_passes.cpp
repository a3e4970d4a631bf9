#include "optimization/graph_passes.h"

namespace fluidml {
namespace optimization {

namespace {

using graph::Edge;
using graph::Graph;
using graph::Node;
using EdgePtr = std::shared_ptr<Edge>;
using NodePtr = std::shared_ptr<Node>;

// an intermediate value: produced and consumed inside the graph
bool IsPure(const EdgePtr &e) { return e != nullptr && e->GetKind() == Edge::Kind::Pure; }

// the single output value of `node`, or nullptr
EdgePtr OnlyOutput(const Graph &g, const NodePtr &node) {
  const std::vector<EdgePtr> outs = g.GetNodeTo(node->GetName());
  return outs.size() == 1 ? outs[0] : nullptr;
}

// the single consumer of the intermediate value `edge`, or nullptr
NodePtr OnlyConsumer(const Graph &g, const EdgePtr &edge) {
  if (!IsPure(edge)) return nullptr;
  const std::vector<NodePtr> to = g.GetEdgeTo(edge->GetName());
  return to.size() == 1 ? to[0] : nullptr;
}

// Replaces `chain` (its intermediate values `dead`) by a node `op` named after the chain members, reading
// `inputs` in that order and producing `output`.
void Replace(Graph &g, const std::vector<NodePtr> &chain, const std::vector<EdgePtr> &dead, Node::Op op,
             const std::vector<EdgePtr> &inputs, const EdgePtr &output) {
  std::string name;
  for (const NodePtr &n : chain) name += (name.empty() ? "" : "-") + n->GetName();
  for (const EdgePtr &e : dead) g.DeleteEdge(e->GetName());
  for (const NodePtr &n : chain) g.DeleteNode(n->GetName());
  const std::string fused = name;
  g.PutNode(std::make_shared<Node>(std::move(name), op));
  for (const EdgePtr &e : inputs) g.EdgeToNode(e->GetName(), fused);
  g.NodeToEdge(fused, output->GetName());
}

}  // namespace

void AddDivErfAddMulFusionPass::Run(Graph &g, const std::string &node_name) const {
  const NodePtr add0 = g.GetNode(node_name);
  if (!add0 || add0->GetOp() != Node::Op::Add) return;
  std::vector<EdgePtr> in = g.GetNodeFrom(node_name);
  if (in.size() != 2) return;
  EdgePtr bias = in[0], x = in[1];
  if (IsPure(bias) && x->IsConstantTensor()) std::swap(bias, x);
  if (!bias->IsConstantTensor() || !IsPure(x)) return;
  const EdgePtr t = OnlyOutput(g, add0);
  if (!IsPure(t)) return;
  const std::vector<NodePtr> readers = g.GetEdgeTo(t->GetName());
  if (readers.size() != 2) return;
  NodePtr mul0 = readers[0], div = readers[1];
  if (mul0->GetOp() == Node::Op::Div && div->GetOp() == Node::Op::Mul) std::swap(mul0, div);
  if (mul0->GetOp() != Node::Op::Mul || div->GetOp() != Node::Op::Div) return;
  const std::vector<EdgePtr> div_in = g.GetNodeFrom(div->GetName());
  if (div_in.size() != 2 || div_in[0] != t || !div_in[1]->IsConstantScalar()) return;
  const EdgePtr div_out = OnlyOutput(g, div);
  const NodePtr erf = OnlyConsumer(g, div_out);
  if (!erf || erf->GetOp() != Node::Op::Erf) return;
  const EdgePtr erf_out = OnlyOutput(g, erf);
  const NodePtr add1 = OnlyConsumer(g, erf_out);
  if (!add1 || add1->GetOp() != Node::Op::Add) return;
  const std::vector<EdgePtr> add1_in = g.GetNodeFrom(add1->GetName());
  if (add1_in.size() != 2 || add1_in[0] != erf_out || !add1_in[1]->IsConstantScalar()) return;
  const EdgePtr add1_out = OnlyOutput(g, add1);
  if (OnlyConsumer(g, add1_out) != mul0) return;
  const EdgePtr mul0_out = OnlyOutput(g, mul0);
  const NodePtr mul1 = OnlyConsumer(g, mul0_out);
  if (!mul1 || mul1->GetOp() != Node::Op::Mul) return;
  const std::vector<EdgePtr> mul1_in = g.GetNodeFrom(mul1->GetName());
  if (mul1_in.size() != 2 || mul1_in[0] != mul0_out || !mul1_in[1]->IsConstantScalar()) return;
  const EdgePtr out = OnlyOutput(g, mul1);
  if (!out) return;
  Replace(g, {add0, div, erf, add1, mul0, mul1}, {t, div_out, erf_out, add1_out, mul0_out}, Node::Op::AddDivErfAddMulMul,
          {bias, div_in[1], add1_in[1], mul1_in[1], x}, out);
}

void GatherAddFusionPass::Run(Graph &g, const std::string &node_name) const {
  const NodePtr gather = g.GetNode(node_name);
  if (!gather || gather->GetOp() != Node::Op::Gather) return;
  const std::vector<EdgePtr> in = g.GetNodeFrom(node_name);
  if (in.size() != 2 || !in[0]->IsConstantTensor() || !in[1]->IsNonConstant()) return;
  if (gather->HasAttribute("axis") && gather->GetAttribute("axis").GetInt64() != 0) return;
  const EdgePtr g_out = OnlyOutput(g, gather);
  const NodePtr add0 = OnlyConsumer(g, g_out);
  if (!add0 || add0->GetOp() != Node::Op::Add) return;
  const std::vector<EdgePtr> add0_in = g.GetNodeFrom(add0->GetName());
  if (add0_in.size() != 2 || add0_in[0] != g_out || !add0_in[1]->IsConstantTensor()) return;
  const EdgePtr add0_out = OnlyOutput(g, add0);
  const NodePtr add1 = OnlyConsumer(g, add0_out);
  if (!add1 || add1->GetOp() != Node::Op::Add) return;
  const std::vector<EdgePtr> add1_in = g.GetNodeFrom(add1->GetName());
  if (add1_in.size() != 2 || add1_in[0] != add0_out || !add1_in[1]->IsConstantTensor()) return;
  const EdgePtr out = OnlyOutput(g, add1);
  if (!out) return;
  Replace(g, {gather, add0, add1}, {g_out, add0_out}, Node::Op::GatherAddAdd, {in[0], add0_in[1], add1_in[1], in[1]}, out);
}

void UnsqueezeSubMulPass::Run(Graph &g, const std::string &node_name) const {
  const NodePtr unsqueeze = g.GetNode(node_name);
  if (!unsqueeze || unsqueeze->GetOp() != Node::Op::Unsqueeze) return;
  const std::vector<EdgePtr> in = g.GetNodeFrom(node_name);
  if (in.size() != 2 || !in[1]->IsConstantTensor()) return;
  const EdgePtr u_out = OnlyOutput(g, unsqueeze);
  const NodePtr sub = OnlyConsumer(g, u_out);
  if (!sub || sub->GetOp() != Node::Op::Sub) return;
  const std::vector<EdgePtr> sub_in = g.GetNodeFrom(sub->GetName());
  if (sub_in.size() != 2 || !sub_in[0]->IsConstantScalar() || sub_in[1] != u_out) return;
  const EdgePtr sub_out = OnlyOutput(g, sub);
  const NodePtr mul = OnlyConsumer(g, sub_out);
  if (!mul || mul->GetOp() != Node::Op::Mul) return;
  const std::vector<EdgePtr> mul_in = g.GetNodeFrom(mul->GetName());
  if (mul_in.size() != 2 || mul_in[0] != sub_out || !mul_in[1]->IsConstantScalar()) return;
  const EdgePtr out = OnlyOutput(g, mul);
  if (!out) return;
  Replace(g, {unsqueeze, sub, mul}, {u_out, sub_out}, Node::Op::UnsqueezeSubMul, {in[1], sub_in[0], mul_in[1], in[0]}, out);
}

void GraphPassesManager::RegisterAllPasses() {
  passes_.push_back(AddDivErfAddMulFusionPass::Make());
  passes_.push_back(GatherAddFusionPass::Make());
  passes_.push_back(UnsqueezeSubMulPass::Make());
}

void GraphPassesManager::Run(Graph &graph) const {
  std::vector<std::string> names;
  for (const std::shared_ptr<Node> &n : graph.GetAllNodes()) names.push_back(n->GetName());
  for (const std::string &name : names) {
    for (const std::shared_ptr<GraphPass> &pass : passes_) {
      if (graph.ExistNode(name)) pass->Run(graph, name);
    }
  }
}

}  // namespace optimization
}  // namespace fluidml
