#include "worker/lower.h"

#include "worker/launcher.h"

namespace fluidml {
namespace worker {
namespace {
class LowerImpl : public Lower {
 public:
  explicit LowerImpl(context::Context &&context) : context_(std::move(context)) {}
  void Run() override { context_->GetModule().Validate(); }

 private:
  context::Context context_;
};
}  // namespace

std::unique_ptr<Lower> Lower::Make(context::Context &&context) { return std::make_unique<LowerImpl>(std::move(context)); }

}  // namespace worker
}  // namespace fluidml
