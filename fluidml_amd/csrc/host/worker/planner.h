// Execution order, lifetimes and the arena plan (reference include/worker/planner.h,
// src/worker/planner.cpp).
#ifndef FLUIDML_AMD_HOST_WORKER_PLANNER_H_
#define FLUIDML_AMD_HOST_WORKER_PLANNER_H_

#include <memory>
#include <string>
#include <tuple>

#include "structure/flow/flow.h"
#include "structure/memory/memory.h"

namespace fluidml {
namespace evaluation {
class DynamicProgrammingTable;
}
namespace worker {

// Kahn's algorithm exactly as the reference runs it (planner.cpp:22-108): the
// ready list is a stack, it is seeded in Flow::GetNodes() order, and after each
// pop the predecessor multimap is scanned from its beginning, so which of
// several ready nodes runs first is decided by libstdc++'s unordered-container
// iteration order over the value and node names.  Node indices of this order
// are the lifetimes of the memory plan.
flow::Sequence TopologicalSort(const flow::Flow &flow);

// Fills `infos` in the reference's order (planner.cpp:236-293): every region
// that needs arena bytes in Sequence::GetRegions() order with lifetime
// [min, max] node index over its Memory edges, then every node with scratch
// under the node's own name with lifetime [i, i].
void CollectInfos(const flow::Sequence &sequence, memory::Infos &infos);

class Planner {
 public:
  virtual ~Planner() = default;
  // (sequence, arena index, layout-DP report as JSON text or "null")
  virtual std::tuple<flow::Sequence, memory::Index, std::string> Run(const flow::Flow &flow) = 0;
  static std::unique_ptr<Planner> MakePlainLinearPlanner();
  static std::unique_ptr<Planner> MakePlainGreedyPlanner();
  // `table` supplies the layout DP; it is run on the flow and its layouts are
  // written into the regions before the arena is planned (planner.cpp:300-320)
  static std::unique_ptr<Planner> MakeDPGreedyPlanner(std::shared_ptr<evaluation::DynamicProgrammingTable> table);
};

}  // namespace worker
}  // namespace fluidml

#endif
