// Graph-level fusion passes (reference include/optimization/graph/{pass,manager,
// add_div_erf_add_mul_fusion,gather_add_fusion,unsqueeze_sub_mul_fusion}.h).
// Each pass looks at one node and, when that node heads the pattern, replaces the
// whole chain by one fused node whose inputs are the chain's constants followed
// by its variable input -- the order the converter of the fused operators reads.
// The reference ships these passes without calling them from Executor::Compile;
// here they run between parsing and conversion when Context::graph_passes is set
// (environment FLUIDML_GRAPH_PASSES=1).  They change the node sequence and
// therefore the memory plan, unlike the launcher's fusion which changes neither.
#ifndef FLUIDML_AMD_HOST_OPTIMIZATION_GRAPH_PASSES_H_
#define FLUIDML_AMD_HOST_OPTIMIZATION_GRAPH_PASSES_H_

#include <memory>
#include <string>
#include <vector>

#include "structure/graph/graph.h"

namespace fluidml {
namespace optimization {

class GraphPass {
 public:
  virtual ~GraphPass() = default;
  // `node_name` names a node of `graph`; the pass may delete it and others
  virtual void Run(graph::Graph &graph, const std::string &node_name) const = 0;
};

// Add(bias) -> Div -> Erf -> Add -> Mul(with the first Add) -> Mul  =>  AddDivErfAddMulMul
// (reference src/optimization/graph/add_div_erf_add_mul_fusion.cpp:16-245)
class AddDivErfAddMulFusionPass : public GraphPass {
 public:
  static std::shared_ptr<AddDivErfAddMulFusionPass> Make() { return std::make_shared<AddDivErfAddMulFusionPass>(); }
  void Run(graph::Graph &graph, const std::string &node_name) const override;
};

// Gather(constant table) -> Add(constant) -> Add(constant)  =>  GatherAddAdd
// (reference src/optimization/graph/gather_add_fusion.cpp:16-135)
class GatherAddFusionPass : public GraphPass {
 public:
  static std::shared_ptr<GatherAddFusionPass> Make() { return std::make_shared<GatherAddFusionPass>(); }
  void Run(graph::Graph &graph, const std::string &node_name) const override;
};

// Unsqueeze -> Sub(scalar - x) -> Mul(scalar)  =>  UnsqueezeSubMul
// (reference src/optimization/graph/unsqueeze_sub_mul_fusion.cpp:17-148)
class UnsqueezeSubMulPass : public GraphPass {
 public:
  static std::shared_ptr<UnsqueezeSubMulPass> Make() { return std::make_shared<UnsqueezeSubMulPass>(); }
  void Run(graph::Graph &graph, const std::string &node_name) const override;
};

// reference src/optimization/graph/manager.cpp:12-34
class GraphPassesManager {
 public:
  GraphPassesManager() = default;
  void RegisterAllPasses();
  void Register(std::shared_ptr<GraphPass> pass) { passes_.push_back(std::move(pass)); }
  // every pass on every node of a snapshot of the node list, in container order
  void Run(graph::Graph &graph) const;

 private:
  std::vector<std::shared_ptr<GraphPass>> passes_;
};

}  // namespace optimization
}  // namespace fluidml

#endif
