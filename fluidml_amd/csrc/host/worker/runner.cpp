#include "worker/runner.h"

#include <stdexcept>

#include "worker/launcher.h"

namespace fluidml {
namespace worker {
namespace {

class RunnerImpl : public Runner {
 public:
  explicit RunnerImpl(context::Context &&context) : context_(std::move(context)) {}

  size_t Run(const std::unordered_map<std::string, void *> &args, size_t epoch) override {
    LaunchPlan &plan = context_->GetModule();
    for (const context::ArgumentAttr &arg : context_->GetFuncAttr().GetArguments()) {
      if (args.at(arg.GetName()) == nullptr) throw std::invalid_argument("Runner: null buffer for " + arg.GetName());
    }
    return plan.Run(args, epoch);
  }

#ifdef BUILD_PYTHON
  size_t Run(const std::unordered_map<std::string, pybind11::array> &args, size_t epoch) override {
    std::unordered_map<std::string, void *> raw;
    for (const context::ArgumentAttr &arg : context_->GetFuncAttr().GetArguments()) {
      const pybind11::array &array = args.at(arg.GetName());
      pybind11::buffer_info info = array.request();
      const size_t bytes = static_cast<size_t>(info.size) * static_cast<size_t>(info.itemsize);
      if (bytes != arg.GetMeta().GetSize()) {
        throw std::invalid_argument("Runner: array for '" + arg.GetName() + "' has " + std::to_string(bytes) +
                                    " bytes, the graph expects " + std::to_string(arg.GetMeta().GetSize()));
      }
      if (!(array.flags() & pybind11::array::c_style)) {
        throw std::invalid_argument("Runner: array for '" + arg.GetName() + "' must be C-contiguous");
      }
      raw.insert({arg.GetName(), info.ptr});
    }
    return Run(raw, epoch);
  }
#endif

 private:
  context::Context context_;
};

}  // namespace

std::unique_ptr<Runner> Runner::Make(context::Context &&context) { return std::make_unique<RunnerImpl>(std::move(context)); }

}  // namespace worker
}  // namespace fluidml
