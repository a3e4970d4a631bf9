// Shared state of one compilation: the launch plan ("module"), its function
// attributes and the options of this backend (reference
// include/structure/context/{context,attr}.h).  `Context` is a cheap handle;
// every worker made from it sees the same ContextImpl.
#ifndef FLUIDML_AMD_HOST_STRUCTURE_CONTEXT_CONTEXT_H_
#define FLUIDML_AMD_HOST_STRUCTURE_CONTEXT_CONTEXT_H_

#include <memory>
#include <optional>
#include <ostream>
#include <string>
#include <vector>

#include "structure/kernel/tuner.h"
#include "structure/tensor/meta.h"

namespace fluidml {
namespace worker {
class GeneralBuilder;
class KernelBuilder;
class Planner;
class Lower;
class Runner;
class LaunchPlan;
}  // namespace worker
namespace evaluation {
class DynamicProgrammingTable;
class CostModel;
}  // namespace evaluation

namespace context {

// One interface tensor of the compiled function (reference attr.h:13-36).
class ArgumentAttr {
 public:
  enum class Type { Input, Output };
  ArgumentAttr(Type type, std::string &&name, Meta &&meta) : type_(type), name_(std::move(name)), meta_(std::move(meta)) {}
  Type GetType() const { return type_; }
  const std::string &GetName() const { return name_; }
  const Meta &GetMeta() const { return meta_; }

 private:
  Type type_;
  std::string name_;
  Meta meta_;
};

// Name, arena bytes and argument list of the compiled function (reference attr.h:38-58).
class FuncAttr {
 public:
  FuncAttr(std::string &&name, size_t buffer) : name_(std::move(name)), buffer_(buffer) {}
  const std::string &GetName() const { return name_; }
  size_t GetBuffer() const { return buffer_; }
  const std::vector<ArgumentAttr> &GetArguments() const { return arguments_; }
  void PutArgument(ArgumentAttr &&arg) { arguments_.push_back(std::move(arg)); }

 private:
  std::string name_;
  size_t buffer_;
  std::vector<ArgumentAttr> arguments_;
};

// How the layout DP obtains kernel costs.
enum class CostMode {
  Measure,   // time every (kernel, layouts) on the GPU with hipEvents
  Constant,  // every cost is 1 (the reference's DP_DEBUG build, eval.cpp:73-76)
  Table      // read costs from a JSON cost table written by an earlier compile
};

class ContextImpl {
 public:
  ContextImpl();
  ~ContextImpl();
  worker::LaunchPlan &GetModule();
  bool HasModule() const { return module_ != nullptr; }
  void SetModule(std::unique_ptr<worker::LaunchPlan> &&module);
  std::unique_ptr<worker::LaunchPlan> ReleaseModule();
  FuncAttr &GetFuncAttr();
  void SetFuncAttr(FuncAttr &&attr);
  // reads "contraction_table" and "side_branches" of a JSON file an earlier Executor::Compile wrote
  void LoadSavedDecisions(const std::string &path);

  // FL_REF_* literal-reference switches (env FLUIDML_REF_QUIRKS=<int>, default 0)
  uint32_t ref_flags = 0;
  // replay the plan as a captured hipGraph (env FLUIDML_HIP_GRAPH=0 disables)
  bool use_graph = true;
  // launch-level fusion of single-reader kernel chains (env FLUIDML_FUSE=0 disables)
  bool fuse = true;
  // run the graph-level fusion passes between parsing and conversion (env FLUIDML_GRAPH_PASSES=1);
  // the reference ships them unwired, so the default is off
  bool graph_passes = false;
  // MatMul nodes on the opt-in bf16 path (env FLUIDML_BF16=1)
  bool bf16 = false;
  // two independent runs of launches go side by side on two streams when the shorter one is estimated at least
  // this long, in microseconds (env FLUIDML_BRANCHES=0 never; negative: the launch plan's default)
  double branch_min_us = -1.0;
  // time the first replays with and without the side branches and keep the faster schedule (env FLUIDML_BRANCH_CHECK=0:
  // keep every candidate region)
  bool branch_check = true;
  // cost source of the layout DP (env FLUIDML_DP_COST=measure|constant|<path to table json>)
  CostMode cost_mode = CostMode::Measure;
  std::string cost_table_path;
  // DP executor with measured costs: time the proposed plan as a whole against the default layouts and keep the
  // faster (env FLUIDML_DP_CHECK=0 keeps the DP's proposal whatever it costs)
  bool dp_check_whole_plan = true;
  std::shared_ptr<evaluation::CostModel> cost_model;  // created on first use
  // Tile configuration per contraction signature, shared by the kernel generators and the launch plan (the
  // reference keeps the equivalent cache inside each MatMul / Gemm generator, generator/matmul.cpp:94-98).
  // Mode from the environment (FLUIDML_TUNE: 0 = the library's rule, a file = replay that compile's table);
  // a cost table given through FLUIDML_DP_COST that carries a "contraction_table" is replayed as well.
  std::shared_ptr<kernel::ContractionTable> contraction_table;
  // side branches of the launch plan: 1 / 0 = keep / drop them without timing (read back from a saved JSON),
  // negative = let the first run decide by timing
  int branch_decision = -1;

 private:
  std::unique_ptr<worker::LaunchPlan> module_;
  std::optional<FuncAttr> func_attr_;
};

class Context {
 public:
  Context();
  ContextImpl &operator*() { return *impl_; }
  ContextImpl *operator->() { return impl_.get(); }
  std::unique_ptr<evaluation::DynamicProgrammingTable> MakeDynamicProgrammingTable();
  std::unique_ptr<worker::GeneralBuilder> MakePlainGeneralBuilder(std::string &&function_name);
  std::unique_ptr<worker::GeneralBuilder> MakeDPGeneralBuilder(std::string &&function_name);
  std::unique_ptr<worker::KernelBuilder> MakeKernelBuilder(std::string &&function_name);
  std::unique_ptr<worker::Planner> MakePlainLinearPlanner();
  std::unique_ptr<worker::Planner> MakePlainGreedyPlanner();
  std::unique_ptr<worker::Planner> MakeDPGreedyPlanner();
  std::unique_ptr<worker::Lower> MakeLower();
  std::unique_ptr<worker::Runner> MakeRunner();
  // textual dump of the launch plan (what `*mlir << context_` prints in the
  // reference, executor.cpp:106-112)
  friend std::ostream &operator<<(std::ostream &os, Context &context);

 private:
  std::shared_ptr<ContextImpl> impl_;
};

}  // namespace context
}  // namespace fluidml

#endif
