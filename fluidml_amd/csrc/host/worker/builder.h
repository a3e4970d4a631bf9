// Builders turn planned flows into launch plans (reference include/worker/builder.h,
// src/worker/builder.cpp).  GeneralBuilder handles a whole sequence;
// KernelBuilder wraps ONE kernel so its cost can be measured.
#ifndef FLUIDML_AMD_HOST_WORKER_BUILDER_H_
#define FLUIDML_AMD_HOST_WORKER_BUILDER_H_

#include <memory>
#include <string>
#include <vector>

#include "structure/context/context.h"
#include "structure/flow/flow.h"
#include "structure/kernel/kernel.h"
#include "structure/memory/memory.h"

namespace fluidml {
namespace worker {

class Builder {
 public:
  virtual ~Builder() = default;
};

class GeneralBuilder : public Builder {
 public:
  // Lays every inner region at its arena offset with its layout's strides,
  // registers constants and interface tensors, places node scratch under
  // Index::Get(node name) and appends one step per node in sequence order
  // (reference builder.cpp:149-394).  Stores the plan and its FuncAttr in the
  // context.
  virtual void Run(const flow::Sequence &sequence, const memory::Index &index) = 0;
  // kernels from SelectKernel(node) (reference builder.cpp:400-491)
  static std::unique_ptr<GeneralBuilder> MakePlain(std::string &&function_name, context::Context &&context);
  // kernels from the node's generator, told the regions' layouts (reference builder.cpp:493-608)
  static std::unique_ptr<GeneralBuilder> MakeDynamicProgramming(std::string &&function_name, context::Context &&context);
};

class KernelBuilder : public Builder {
 public:
  // Each call replaces the context's module with a one-step plan whose
  // operands are interface tensors named by the keys below (reference
  // builder.cpp:637-960).  Without layouts the identity layout is used.
  virtual void RunOnSingleInputWithoutBuffer(std::shared_ptr<kernel::SingleInputWithoutBufferKernel> kernel,
                                             const Meta &input_meta, const std::vector<size_t> &input_layout,
                                             const Meta &output_meta, const std::vector<size_t> &output_layout) = 0;
  virtual void RunOnSingleInputWithBuffer(std::shared_ptr<kernel::SingleInputWithBufferKernel> kernel,
                                          const Meta &input_meta, const std::vector<size_t> &input_layout,
                                          const Meta &output_meta, const std::vector<size_t> &output_layout,
                                          size_t buffer_size) = 0;
  virtual void RunOnDoubleInputsWithoutBuffer(std::shared_ptr<kernel::DoubleInputsWithoutBufferKernel> kernel,
                                              const Meta &lhs_meta, const std::vector<size_t> &lhs_layout,
                                              const Meta &rhs_meta, const std::vector<size_t> &rhs_layout,
                                              const Meta &output_meta, const std::vector<size_t> &output_layout) = 0;
  virtual void RunOnDoubleInputsWithBuffer(std::shared_ptr<kernel::DoubleInputsWithBufferKernel> kernel,
                                           const Meta &lhs_meta, const std::vector<size_t> &lhs_layout,
                                           const Meta &rhs_meta, const std::vector<size_t> &rhs_layout,
                                           const Meta &output_meta, const std::vector<size_t> &output_layout,
                                           size_t buffer_size) = 0;
  static constexpr char kInputKey[] = "input";
  static constexpr char kLhsKey[] = "lhs";
  static constexpr char kRhsKey[] = "rhs";
  static constexpr char kOutputKey[] = "output";
  static std::unique_ptr<KernelBuilder> Make(std::string &&function_name, context::Context &&context);
};

}  // namespace worker
}  // namespace fluidml

#endif
