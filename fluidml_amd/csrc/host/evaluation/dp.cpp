#include "evaluation/dp.h"

#include <algorithm>
#include <deque>
#include <limits>
#include <map>
#include <stdexcept>
#include <unordered_set>

#include "evaluation/eval.h"
#include "utils/json.h"
#include "utils/utils.h"

namespace fluidml {
namespace evaluation {

namespace {

using EdgePtr = std::shared_ptr<flow::Edge>;
using NodePtr = std::shared_ptr<flow::Node>;

bool FromOutside(const EdgePtr &e) {
  return e->GetKind() == flow::Edge::Kind::Input || e->GetKind() == flow::Edge::Kind::Constant;
}

EdgePtr MakeInputEdge(const EdgePtr &like, const NodePtr &to) {
  return std::make_shared<flow::Edge>(flow::Edge::Kind::Input, std::shared_ptr<flow::Region>(like->GetRegion()), nullptr,
                                      NodePtr(to));
}

EdgePtr MakeOutputEdge(const EdgePtr &like, const NodePtr &from) {
  return std::make_shared<flow::Edge>(flow::Edge::Kind::Output, std::shared_ptr<flow::Region>(like->GetRegion()),
                                      NodePtr(from), nullptr);
}

// An insertion-ordered set.  The reference keeps these sets keyed by object
// address (std::unordered_set<std::shared_ptr<...>>, dp.cpp:159,165-166,240-242),
// which makes its subflow order differ from run to run; here every such set
// iterates in insertion order, which is a function of the flow's name-keyed
// containers only.
template <typename T>
class OrderedSet {
 public:
  bool Insert(const T &v) {
    if (!seen_.insert(v.get()).second) return false;
    items_.push_back(v);
    return true;
  }
  bool Contains(const T &v) const { return seen_.count(v.get()) > 0; }
  const std::vector<T> &Items() const { return items_; }

 private:
  std::vector<T> items_;
  std::unordered_set<const void *> seen_;
};

// Splits a flow into chains the DP can solve: the longest path first, then the
// remaining nodes grouped into connected branches, each split again
// (reference SubFlowsBuilder, dp.cpp:137-568).
class SubFlowsBuilder {
 public:
  std::vector<flow::Flow> Run(const flow::Flow &flow) {
    std::vector<flow::Flow> subflows;
    const std::vector<EdgePtr> edges = flow.GetEdges();
    const std::vector<NodePtr> nodes = flow.GetNodes();
    if (nodes.empty()) return subflows;
    std::unordered_map<std::string, Reach> table;
    size_t farthest_distance = 0;
    EdgePtr farthest_edge;
    for (const EdgePtr &edge : edges) {
      const size_t distance = LongestPathTo(flow, table, edge);
      if (distance > farthest_distance) {  // strict: the first farthest edge in container order wins
        farthest_distance = distance;
        farthest_edge = edge;
      }
    }
    if (!farthest_edge) throw std::logic_error("layout DP: flow without a computed edge");

    // ---- main chain: every edge on the longest path, each consumer node, and
    // for a double-input consumer its off-path operand as a fresh Input edge ----
    std::vector<EdgePtr> path;
    for (EdgePtr e = farthest_edge; e; e = table.at(e->GetName()).prev) path.push_back(e);
    flow::Flow main_subflow;
    OrderedSet<NodePtr> main_nodes;
    OrderedSet<EdgePtr> main_edges;
    for (const EdgePtr &edge : path) {
      if (edge->OwnsTo()) {
        const NodePtr &to = edge->GetTo();
        if (to->IsDoubleInputs()) {
          const EdgePtr lhs = flow.GetLhsEdge(*to), rhs = flow.GetRhsEdge(*to);
          EdgePtr off_path;
          if (lhs == edge) off_path = rhs;
          else if (rhs == edge) off_path = lhs;
          else throw std::logic_error("layout DP: path edge is not an operand of its consumer");
          main_edges.Insert(MakeInputEdge(off_path, to));
        }
        main_nodes.Insert(to);
      }
      main_edges.Insert(edge);
    }
    for (const NodePtr &node : main_nodes.Items()) main_subflow.PutNode(NodePtr(node));
    for (const EdgePtr &edge : main_edges.Items()) {
      if (!main_subflow.GetRegion(edge->GetName())) main_subflow.PutRegion(std::shared_ptr<flow::Region>(edge->GetRegion()));
      main_subflow.PutEdge(EdgePtr(edge));
    }
    subflows.push_back(std::move(main_subflow));

    // ---- branches: connected groups of the nodes that are left ----
    OrderedSet<NodePtr> assigned;
    std::vector<std::vector<NodePtr>> branches;
    for (const NodePtr &seed : nodes) {
      if (main_nodes.Contains(seed) || assigned.Contains(seed)) continue;
      OrderedSet<NodePtr> branch;
      std::deque<NodePtr> frontier{seed};
      while (!frontier.empty()) {
        NodePtr node = frontier.front();
        frontier.pop_front();
        if (branch.Contains(node)) continue;
        auto visit = [&](const NodePtr &other) {
          if (other && !main_nodes.Contains(other) && !branch.Contains(other)) frontier.push_back(other);
        };
        const EdgePtr lhs = flow.GetLhsEdge(*node), out = flow.GetOutputEdge(*node);
        if (lhs->OwnsFrom()) visit(lhs->GetFrom());
        if (node->IsDoubleInputs()) {
          const EdgePtr rhs = flow.GetRhsEdge(*node);
          if (rhs->OwnsFrom()) visit(rhs->GetFrom());
        }
        if (out->OwnsTo()) visit(out->GetTo());
        branch.Insert(node);
        assigned.Insert(node);
      }
      branches.push_back(branch.Items());
    }
    for (const std::vector<NodePtr> &branch_nodes : branches) {
      std::unordered_set<const flow::Node *> in_branch;
      for (const NodePtr &n : branch_nodes) in_branch.insert(n.get());
      flow::Flow branch;
      auto put_region = [&](const EdgePtr &e) {
        if (!branch.GetRegion(e->GetName())) branch.PutRegion(std::shared_ptr<flow::Region>(e->GetRegion()));
      };
      auto put_edge = [&](const EdgePtr &e) {
        const std::vector<EdgePtr> same_name = branch.GetEdges(e->GetName());
        if (std::find(same_name.begin(), same_name.end(), e) == same_name.end()) branch.PutEdge(EdgePtr(e));
      };
      // an operand produced outside the branch becomes an Input edge, a result
      // consumed outside becomes an Output edge (reference dp.cpp:350-398)
      auto operand = [&](const EdgePtr &e, const NodePtr &node) {
        if (e->IsMemory() && !in_branch.count(e->GetFrom().get())) return MakeInputEdge(e, node);
        return e;
      };
      for (const NodePtr &node : branch_nodes) {
        std::vector<EdgePtr> ins{operand(flow.GetLhsEdge(*node), node)};
        if (node->IsDoubleInputs()) ins.push_back(operand(flow.GetRhsEdge(*node), node));
        EdgePtr out = flow.GetOutputEdge(*node);
        if (out->IsMemory() && !in_branch.count(out->GetTo().get())) out = MakeOutputEdge(out, node);
        for (const EdgePtr &e : ins) put_region(e);
        put_region(out);
        branch.PutNode(NodePtr(node));
        for (const EdgePtr &e : ins) put_edge(e);
        put_edge(out);
      }
      for (flow::Flow &sub : SubFlowsBuilder().Run(branch)) subflows.push_back(std::move(sub));
    }
    return subflows;
  }

 private:
  struct Reach {
    size_t distance;
    EdgePtr prev;
  };
  // Unit-weight longest path from any outside edge to `edge`, memoised by
  // region name; between two operands the right one wins a tie
  // (reference dp.cpp:570-669).
  size_t LongestPathTo(const flow::Flow &flow, std::unordered_map<std::string, Reach> &table, const EdgePtr &edge) {
    auto it = table.find(edge->GetName());
    if (it != table.end()) return it->second.distance;
    size_t distance = 0;
    EdgePtr prev;
    if (!FromOutside(edge)) {
      const NodePtr &from = edge->GetFrom();
      if (from->IsSingleInput()) {
        prev = flow.GetInputEdge(*from);
        distance = LongestPathTo(flow, table, prev) + 1;
      } else {
        const EdgePtr lhs = flow.GetLhsEdge(*from), rhs = flow.GetRhsEdge(*from);
        const size_t l = LongestPathTo(flow, table, lhs), r = LongestPathTo(flow, table, rhs);
        if (l > r) {
          distance = l + 1;
          prev = lhs;
        } else {
          distance = r + 1;
          prev = rhs;
        }
      }
    }
    table.insert({edge->GetName(), Reach{distance, prev}});
    return distance;
  }
};

// Minimum-cost layout assignment on one chain-shaped subflow
// (reference DPOnNoOverlapFlowWoker, dp.cpp:695-842).
class ChainSolver {
 public:
  explicit ChainSolver(std::shared_ptr<worker::Evaluator> evaluator) : evaluator_(std::move(evaluator)) {}

  DynamicProgrammingPlan Run(const flow::Flow &flow) {
    std::unordered_map<std::string, Layout> chosen;
    for (const EdgePtr &edge : flow.GetEdges()) {
      if (edge->GetKind() != flow::Edge::Kind::Output) continue;
      // Every layout of the result is solved, in enumeration order, but the
      // table keeps the first value written per tensor: the result tensor ends
      // up with GenAllOrders(rank)[0] and the chain with the best layouts
      // *for that* (reference dp.cpp:705-733).
      for (const Layout &layout : utils::GenAllOrders(edge->GetLayout().size())) {
        Solve(flow, edge, layout);
        std::deque<Key> queue{Key{edge.get(), layout}};
        chosen.insert({edge->GetName(), layout});
        while (!queue.empty()) {
          const Key at = queue.front();
          queue.pop_front();
          for (const Dep &dep : memo_.at(at).deps) {
            chosen.insert({dep.edge->GetName(), dep.layout});
            queue.push_back(Key{dep.edge.get(), dep.layout});
          }
        }
      }
    }
    return DynamicProgrammingPlan(std::move(chosen));
  }

 private:
  using Key = std::pair<const flow::Edge *, Layout>;
  struct Dep {
    EdgePtr edge;
    Layout layout;
  };
  struct Best {
    size_t cost;
    std::vector<Dep> deps;
  };

  // cost(edge, layout) = min over operand layouts of kernel cost + operand
  // costs; edges from outside cost 0 in any layout; the first minimum in
  // enumeration order wins (strict >, reference dp.cpp:787, 820)
  size_t Solve(const flow::Flow &flow, const EdgePtr &edge, const Layout &layout) {
    const Key key{edge.get(), layout};
    auto it = memo_.find(key);
    if (it != memo_.end()) return it->second.cost;
    Best best{0, {}};
    if (!FromOutside(edge)) {
      const NodePtr &node = edge->GetFrom();
      best.cost = std::numeric_limits<size_t>::max();
      if (node->IsSingleInput()) {
        const EdgePtr input = flow.GetInputEdge(*node);
        KernelEval &eval = evaluator_->GetSingleInputEval(node->GetName());
        for (const Layout &in_layout : utils::GenAllOrders(input->GetMeta().GetShape().size())) {
          const size_t cost = eval.GetTimeCost(in_layout, layout) + Solve(flow, input, in_layout);
          if (best.cost > cost) best = Best{cost, {Dep{input, in_layout}}};
        }
      } else {
        const EdgePtr lhs = flow.GetLhsEdge(*node), rhs = flow.GetRhsEdge(*node);
        KernelEval &eval = evaluator_->GetDoubleInputsEval(node->GetName());
        const auto lhs_layouts = utils::GenAllOrders(lhs->GetMeta().GetShape().size());
        const auto rhs_layouts = utils::GenAllOrders(rhs->GetMeta().GetShape().size());
        for (const Layout &l : lhs_layouts) {
          for (const Layout &r : rhs_layouts) {
            const size_t cost = eval.GetTimeCost(l, r, layout) + Solve(flow, lhs, l) + Solve(flow, rhs, r);
            if (best.cost > cost) best = Best{cost, {Dep{lhs, l}, Dep{rhs, r}}};
          }
        }
      }
    }
    const size_t cost = best.cost;
    memo_.insert({key, std::move(best)});
    return cost;
  }

  std::shared_ptr<worker::Evaluator> evaluator_;
  std::map<Key, Best> memo_;
};

class DynamicProgrammingTableImpl : public DynamicProgrammingTable {
 public:
  explicit DynamicProgrammingTableImpl(std::shared_ptr<CostModel> cost) : cost_(std::move(cost)) {}

  DynamicProgrammingPlan Run(const flow::Flow &flow) override {
    std::vector<flow::Flow> subflows = SubFlowsBuilder().Run(flow);
    DynamicProgrammingPlan plan;
    for (const flow::Flow &subflow : subflows) {
      ChainSolver solver(GetEvaluator(flow));
      plan = Merge(plan, solver.Run(subflow));  // earlier subflows keep their choice
    }
    return plan;
  }

  std::string ToJson() const override {
    return evaluator_ ? "{\"evaluator\":" + evaluator_->ToJson() + "}" : "{}";
  }

 private:
  // one eval per node of the whole flow, shared between nodes of equal kernel
  // kind and metas (reference dp.cpp:914-1018)
  std::shared_ptr<worker::Evaluator> GetEvaluator(const flow::Flow &flow) {
    if (evaluator_) return evaluator_;
    evaluator_ = worker::Evaluator::Make();
    for (const NodePtr &node : flow.GetNodes()) {
      auto generator = std::make_shared<kernel::KernelGenerator>(*node);
      std::string name = node->GetName();
      evaluator_->RegisterEval(std::move(name), std::make_shared<KernelEval>(std::move(generator), cost_));
    }
    return evaluator_;
  }
  std::shared_ptr<CostModel> cost_;
  std::shared_ptr<worker::Evaluator> evaluator_;
};

}  // namespace

DynamicProgrammingPlan::DynamicProgrammingPlan(std::unordered_map<std::string, std::vector<size_t>> &&plan)
    : plan_(std::move(plan)) {}

bool DynamicProgrammingPlan::HasLayout(const std::string &name) const { return plan_.find(name) != plan_.end(); }

const std::vector<size_t> &DynamicProgrammingPlan::GetLayout(const std::string &name) const { return plan_.at(name); }

std::string DynamicProgrammingPlan::ToJson() const {
  std::map<std::string, std::vector<size_t>> sorted(plan_.begin(), plan_.end());
  std::string s = "{";
  bool first = true;
  for (const auto &kv : sorted) {
    s += (first ? "" : ",") + json::Quote(kv.first) + ":[";
    for (size_t i = 0; i < kv.second.size(); ++i) s += (i ? "," : "") + std::to_string(kv.second[i]);
    s += "]";
    first = false;
  }
  return s + "}";
}

DynamicProgrammingPlan Merge(const DynamicProgrammingPlan &lhs, const DynamicProgrammingPlan &rhs) {
  std::unordered_map<std::string, std::vector<size_t>> plan;
  for (const auto &kv : lhs.plan_) plan.insert(kv);
  for (const auto &kv : rhs.plan_) plan.insert(kv);
  return DynamicProgrammingPlan(std::move(plan));
}

std::unique_ptr<DynamicProgrammingTable> DynamicProgrammingTable::Make(std::shared_ptr<CostModel> cost) {
  if (!cost) throw std::invalid_argument("DynamicProgrammingTable::Make: a cost model is required");
  return std::make_unique<DynamicProgrammingTableImpl>(std::move(cost));
}

}  // namespace evaluation
}  // namespace fluidml
