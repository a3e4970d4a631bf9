#include "structure/context/context.h"

#include <cstdlib>
#include <fstream>
#include <sstream>
#include <stdexcept>

#include "utils/json.h"

#include "evaluation/dp.h"
#include "evaluation/eval.h"
#include "worker/builder.h"
#include "worker/launcher.h"
#include "worker/lower.h"
#include "worker/planner.h"
#include "worker/runner.h"

namespace fluidml {
namespace context {

ContextImpl::ContextImpl() {
  if (const char *q = std::getenv("FLUIDML_REF_QUIRKS")) ref_flags = static_cast<uint32_t>(std::strtoul(q, nullptr, 0));
  if (const char *g = std::getenv("FLUIDML_HIP_GRAPH")) use_graph = std::string(g) != "0";
  if (const char *f = std::getenv("FLUIDML_FUSE")) fuse = std::string(f) != "0";
  if (const char *h = std::getenv("FLUIDML_BF16")) bf16 = std::string(h) != "0";
  if (const char *gp = std::getenv("FLUIDML_GRAPH_PASSES")) graph_passes = std::string(gp) != "0";
  if (const char *k = std::getenv("FLUIDML_DP_CHECK")) dp_check_whole_plan = std::string(k) != "0";
  if (const char *c = std::getenv("FLUIDML_DP_COST")) {
    const std::string mode(c);
    if (mode == "constant") {
      cost_mode = CostMode::Constant;
    } else if (mode == "measure" || mode.empty()) {
      cost_mode = CostMode::Measure;
    } else {
      cost_mode = CostMode::Table;
      cost_table_path = mode;
    }
  }
  contraction_table = std::make_shared<kernel::ContractionTable>(kernel::ContractionTable::FromEnvironment());
  // a saved compile replays everything it decided by timing: the layout costs (above), and from the same file the
  // tile configurations and whether the side branches stayed
  std::string saved = cost_mode == CostMode::Table ? cost_table_path : std::string();
  if (const char *t = std::getenv("FLUIDML_TUNE")) {
    const std::string v(t);
    if (!v.empty() && v != "0" && v != "1") saved = v;
  }
  if (!saved.empty()) LoadSavedDecisions(saved);
}

void ContextImpl::LoadSavedDecisions(const std::string &path) {
  std::ifstream ifs(path);
  if (!ifs) return;  // the cost model reports a missing table itself
  std::stringstream text;
  text << ifs.rdbuf();
  const json::Value doc = json::Parse(text.str());
  if (doc.Has("contraction_table") && contraction_table->GetMode() != kernel::ContractionTable::Mode::Off) {
    contraction_table->LoadJson(doc);
    contraction_table->SetMode(kernel::ContractionTable::Mode::Replay);
  }
  if (doc.Has("side_branches") && doc.At("side_branches").Has("kept")) {
    branch_decision = doc.At("side_branches").At("kept").boolean ? 1 : 0;
  }
}

ContextImpl::~ContextImpl() = default;

worker::LaunchPlan &ContextImpl::GetModule() {
  if (!module_) throw std::logic_error("Context: nothing has been built yet (run a GeneralBuilder first)");
  return *module_;
}

void ContextImpl::SetModule(std::unique_ptr<worker::LaunchPlan> &&module) { module_ = std::move(module); }

std::unique_ptr<worker::LaunchPlan> ContextImpl::ReleaseModule() { return std::move(module_); }

FuncAttr &ContextImpl::GetFuncAttr() {
  if (!func_attr_) throw std::logic_error("Context: no function attributes yet (run a builder first)");
  return *func_attr_;
}

void ContextImpl::SetFuncAttr(FuncAttr &&attr) { func_attr_ = std::move(attr); }

Context::Context() : impl_(std::make_shared<ContextImpl>()) {}

std::unique_ptr<evaluation::DynamicProgrammingTable> Context::MakeDynamicProgrammingTable() {
  if (!impl_->cost_model) impl_->cost_model = evaluation::CostModel::Make(*this);
  return evaluation::DynamicProgrammingTable::Make(impl_->cost_model);
}

std::unique_ptr<worker::GeneralBuilder> Context::MakePlainGeneralBuilder(std::string &&function_name) {
  return worker::GeneralBuilder::MakePlain(std::move(function_name), Context(*this));
}
std::unique_ptr<worker::GeneralBuilder> Context::MakeDPGeneralBuilder(std::string &&function_name) {
  return worker::GeneralBuilder::MakeDynamicProgramming(std::move(function_name), Context(*this));
}
std::unique_ptr<worker::KernelBuilder> Context::MakeKernelBuilder(std::string &&function_name) {
  return worker::KernelBuilder::Make(std::move(function_name), Context(*this));
}
std::unique_ptr<worker::Planner> Context::MakePlainLinearPlanner() { return worker::Planner::MakePlainLinearPlanner(); }
std::unique_ptr<worker::Planner> Context::MakePlainGreedyPlanner() { return worker::Planner::MakePlainGreedyPlanner(); }
std::unique_ptr<worker::Planner> Context::MakeDPGreedyPlanner() {
  return worker::Planner::MakeDPGreedyPlanner(MakeDynamicProgrammingTable());
}
std::unique_ptr<worker::Lower> Context::MakeLower() { return worker::Lower::Make(Context(*this)); }
std::unique_ptr<worker::Runner> Context::MakeRunner() { return worker::Runner::Make(Context(*this)); }

std::ostream &operator<<(std::ostream &os, Context &context) {
  if (context->HasModule()) os << context->GetModule().ToText();
  return os;
}

}  // namespace context
}  // namespace fluidml
