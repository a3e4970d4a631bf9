// The reference lowers its MLIR module to LLVM here (src/worker/lower.cpp:38-59).
// A launch plan needs no lowering; this stage keeps its place in the pipeline
// and checks the plan instead (operands inside the arena, names resolvable).
#ifndef FLUIDML_AMD_HOST_WORKER_LOWER_H_
#define FLUIDML_AMD_HOST_WORKER_LOWER_H_

#include <memory>

#include "structure/context/context.h"

namespace fluidml {
namespace worker {

class Lower {
 public:
  virtual ~Lower() = default;
  virtual void Run() = 0;  // throws std::logic_error on an inconsistent plan
  static std::unique_ptr<Lower> Make(context::Context &&context);
};

}  // namespace worker
}  // namespace fluidml

#endif
