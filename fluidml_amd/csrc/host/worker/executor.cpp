#include "worker/executor.h"

#include "optimization/graph_passes.h"

#include <stdexcept>

#include "worker/builder.h"
#include "worker/converter.h"
#include "worker/lower.h"
#include "worker/parser.h"
#include "worker/planner.h"
#include "worker/runner.h"

namespace fluidml {
namespace worker {
namespace {

enum class Flavour { PlainLinear, PlainGreedy, DPGreedy };

class ExecutorImpl : public Executor {
 public:
  ExecutorImpl(std::string &&name, size_t epoch, Flavour flavour)
      : name_(std::move(name)), epoch_(epoch), flavour_(flavour) {}

  void Compile(std::istream &input, std::ofstream *mlir, std::ofstream *llvm, std::ofstream *json) override {
    std::unique_ptr<Parser> parser = Parser::Make();
    std::unique_ptr<Converter> converter = Converter::Make();
    std::string fn = name_;
    std::unique_ptr<GeneralBuilder> builder = flavour_ == Flavour::DPGreedy ? context_.MakeDPGeneralBuilder(std::move(fn))
                                                                            : context_.MakePlainGeneralBuilder(std::move(fn));
    std::unique_ptr<Lower> lower = context_.MakeLower();
    graph::Graph graph = parser->Run(input);
    if (context_->graph_passes) {
      optimization::GraphPassesManager passes;
      passes.RegisterAllPasses();
      passes.Run(graph);
    }
    flow::Flow flow = converter->Run(graph);
    std::unique_ptr<Planner> planner;
    switch (flavour_) {
      case Flavour::PlainLinear: planner = context_.MakePlainLinearPlanner(); break;
      case Flavour::PlainGreedy: planner = context_.MakePlainGreedyPlanner(); break;
      case Flavour::DPGreedy: planner = context_.MakeDPGreedyPlanner(); break;
    }
    auto [sequence, index, dp_json] = planner->Run(flow);
    if (json) *json << dp_json;
    builder->Run(sequence, index);
    if (mlir) *mlir << context_;
    lower->Run();
    if (llvm) *llvm << context_;
  }

  void Compile(std::string_view input, std::optional<std::string_view> mlir, std::optional<std::string_view> llvm,
               std::optional<std::string_view> json) override {
    std::ifstream ifs(std::string(input), std::ios::binary);
    if (!ifs) throw std::runtime_error("Executor::Compile: cannot open " + std::string(input));
    std::ofstream mlir_ofs, llvm_ofs, json_ofs;
    if (mlir) mlir_ofs.open(std::string(*mlir));
    if (llvm) llvm_ofs.open(std::string(*llvm));
    if (json) json_ofs.open(std::string(*json));
    Compile(ifs, mlir ? &mlir_ofs : nullptr, llvm ? &llvm_ofs : nullptr, json ? &json_ofs : nullptr);
  }

  size_t Invoke(const std::unordered_map<std::string, void *> &args) override {
    return context_.MakeRunner()->Run(args, epoch_);
  }

#ifdef BUILD_PYTHON
  size_t Invoke(const std::unordered_map<std::string, pybind11::array> &args) override {
    return context_.MakeRunner()->Run(args, epoch_);
  }
#endif

  context::Context &GetContext() override { return context_; }

 private:
  std::string name_;
  size_t epoch_;
  Flavour flavour_;
  context::Context context_;
};

}  // namespace

std::unique_ptr<Executor> Executor::MakePlainLinear(std::string &&name, size_t epoch) {
  return std::make_unique<ExecutorImpl>(std::move(name), epoch, Flavour::PlainLinear);
}
std::unique_ptr<Executor> Executor::MakePlainGreedy(std::string &&name, size_t epoch) {
  return std::make_unique<ExecutorImpl>(std::move(name), epoch, Flavour::PlainGreedy);
}
std::unique_ptr<Executor> Executor::MakeDPGreedy(std::string &&name, size_t epoch) {
  return std::make_unique<ExecutorImpl>(std::move(name), epoch, Flavour::DPGreedy);
}

}  // namespace worker
}  // namespace fluidml
