#include "worker/planner.h"

#include <algorithm>
#include <list>
#include <stdexcept>
#include <unordered_map>

#include "evaluation/dp.h"

namespace fluidml {
namespace worker {

namespace {
bool FedFromOutside(const std::shared_ptr<flow::Edge> &edge) {
  return edge && (edge->GetKind() == flow::Edge::Kind::Input || edge->GetKind() == flow::Edge::Kind::Constant);
}
}  // namespace

flow::Sequence TopologicalSort(const flow::Flow &flow) {
  flow::Sequence sequence;
  std::unordered_map<std::string, std::shared_ptr<flow::Node>> unvisited;
  std::list<std::shared_ptr<flow::Node>> ready;  // used as a stack
  const std::vector<std::shared_ptr<flow::Node>> nodes = flow.GetNodes();
  const std::vector<std::shared_ptr<flow::Edge>> edges = flow.GetEdges();
  for (const std::shared_ptr<flow::Node> &node : nodes) {
    const bool is_source = node->IsSingleInput()
                               ? FedFromOutside(flow.GetInputEdge(*node))
                               : FedFromOutside(flow.GetLhsEdge(*node)) && FedFromOutside(flow.GetRhsEdge(*node));
    if (is_source) ready.push_back(node);
    else unvisited.insert({node->GetName(), node});
  }
  // consumer name -> producer name, one entry per Memory edge, in edge order
  std::unordered_multimap<std::string, std::string> pending;
  for (const std::shared_ptr<flow::Edge> &edge : edges) {
    if (edge->IsMemory()) pending.insert({edge->GetTo()->GetName(), edge->GetFrom()->GetName()});
  }
  while (!ready.empty()) {
    std::shared_ptr<flow::Node> node = std::move(ready.back());
    ready.pop_back();
    const std::string &name = node->GetName();
    sequence.PutNode(std::shared_ptr<flow::Node>(node));
    for (auto it = pending.begin(); it != pending.end();) {
      if (it->second == name) {
        const std::string consumer = it->first;
        it = pending.erase(it);
        if (pending.find(consumer) == pending.end()) {
          auto found = unvisited.find(consumer);
          if (found == unvisited.end()) throw std::logic_error("TopologicalSort: consumer " + consumer + " released twice");
          ready.push_back(std::move(found->second));
          unvisited.erase(found);
        }
      } else {
        ++it;
      }
    }
  }
  if (!unvisited.empty()) throw std::runtime_error("TopologicalSort: the flow has a cycle or an unfed node");
  for (const std::shared_ptr<flow::Edge> &edge : edges) sequence.PutEdge(std::shared_ptr<flow::Edge>(edge));
  for (const std::shared_ptr<flow::Region> &region : flow.GetRegions()) sequence.PutRegion(std::shared_ptr<flow::Region>(region));
  return sequence;
}

void CollectInfos(const flow::Sequence &sequence, memory::Infos &infos) {
  const auto &nodes = sequence.GetNodes();
  std::unordered_map<std::string, size_t> node_index;
  for (size_t i = 0; i < nodes.size(); ++i) node_index.insert({nodes[i]->GetName(), i});
  std::unordered_multimap<std::string, std::string> users;  // region name -> names of producer and consumers
  for (const std::shared_ptr<flow::Edge> &edge : sequence.GetEdges()) {
    if (edge->IsMemory()) {
      users.insert({edge->GetName(), edge->GetFrom()->GetName()});
      users.insert({edge->GetName(), edge->GetTo()->GetName()});
    }
  }
  for (const std::shared_ptr<flow::Region> &region : sequence.GetRegions()) {
    if (!region->NeedMemoryAllocation()) continue;
    size_t first = static_cast<size_t>(-1), last = 0;
    auto range = users.equal_range(region->GetName());
    for (auto it = range.first; it != range.second; ++it) {
      const size_t i = node_index.at(it->second);
      first = std::min(first, i);
      last = std::max(last, i);
    }
    // A value nobody consumes through a Memory edge keeps (SIZE_MAX, 0), exactly as in the
    // reference's release build (only a DEBUG assert objects, planner.cpp:273-276): it is still
    // queued, it co-lives with nothing and therefore lands at offset 0.  The launcher gives such
    // a region private bytes so that a node writing it cannot clobber the arena.
    std::string name = region->GetName();
    infos.Push(memory::Info(std::move(name), first, last, region->GetMeta().GetSize()));
  }
  for (size_t i = 0; i < nodes.size(); ++i) {
    const size_t scratch = nodes[i]->GetBufferSize();
    if (scratch > 0) {
      std::string name = nodes[i]->GetName();
      infos.Push(memory::Info(std::move(name), i, i, scratch));
    }
  }
}

namespace {

class PlannerImpl : public Planner {
 public:
  PlannerImpl(bool greedy, std::shared_ptr<evaluation::DynamicProgrammingTable> table)
      : greedy_(greedy), table_(std::move(table)) {}

  std::tuple<flow::Sequence, memory::Index, std::string> Run(const flow::Flow &flow) override {
    flow::Sequence sequence = TopologicalSort(flow);
    std::string json = "null";
    if (table_) {
      evaluation::DynamicProgrammingPlan plan = table_->Run(flow);
      for (const std::shared_ptr<flow::Region> &region : sequence.GetRegions()) {
        if (plan.HasLayout(region->GetName())) {
          std::vector<size_t> layout = plan.GetLayout(region->GetName());
          region->SetLayout(std::move(layout));
        }
      }
      json = "{\"dp_table\":" + table_->ToJson() + ",\"plan\":" + plan.ToJson() + "}";
    }
    std::unique_ptr<memory::Infos> infos;
    std::unique_ptr<memory::Plan> plan;
    if (greedy_) {
      infos = std::make_unique<memory::GreedyInfos>();
      plan = std::make_unique<memory::GreedyPlan>();
    } else {
      infos = std::make_unique<memory::PlainInfos>();
      plan = std::make_unique<memory::LinearPlan>();
    }
    CollectInfos(sequence, *infos);
    memory::Index index = plan->Run(*infos);
    return {std::move(sequence), std::move(index), std::move(json)};
  }

 private:
  bool greedy_;
  std::shared_ptr<evaluation::DynamicProgrammingTable> table_;
};

}  // namespace

std::unique_ptr<Planner> Planner::MakePlainLinearPlanner() { return std::make_unique<PlannerImpl>(false, nullptr); }
std::unique_ptr<Planner> Planner::MakePlainGreedyPlanner() { return std::make_unique<PlannerImpl>(true, nullptr); }
std::unique_ptr<Planner> Planner::MakeDPGreedyPlanner(std::shared_ptr<evaluation::DynamicProgrammingTable> table) {
  if (!table) throw std::invalid_argument("MakeDPGreedyPlanner: a DynamicProgrammingTable is required");
  return std::make_unique<PlannerImpl>(true, std::move(table));
}

}  // namespace worker
}  // namespace fluidml
