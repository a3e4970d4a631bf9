// Per-node kernel factories (reference include/structure/kernel/generator/generator.h:11-141).
// A generator knows a node's metas and attributes and yields the kernel for a
// given choice of operand layouts.  On this backend a kernel reads strides
// from its views at launch, so the yielded object does not depend on the
// layouts; the layouts still key the cost cache of the layout DP, and two
// generators that ShapeEquals share one cost-table entry exactly as in the
// reference (generator.cpp:8-42: same generator type and same metas, attributes
// ignored).
#ifndef FLUIDML_AMD_HOST_STRUCTURE_KERNEL_GENERATOR_H_
#define FLUIDML_AMD_HOST_STRUCTURE_KERNEL_GENERATOR_H_

#include <memory>
#include <string>
#include <vector>

#include "structure/flow/flow.h"
#include "structure/kernel/kernel.h"

namespace fluidml {
namespace kernel {

class KernelGenerator {
 public:
  // `node` supplies kind, attributes and the operand metas
  explicit KernelGenerator(const flow::Node &node);
  std::string GetKernelName() const;
  flow::OpKind GetKind() const { return kind_; }
  bool IsSingleInput() const { return !rhs_meta_; }
  bool HasBuffer() const { return has_buffer_; }
  size_t GetBufferSize() const { return buffer_size_; }
  const Meta &GetInputMeta() const { return lhs_meta_; }
  const Meta &GetLhsMeta() const { return lhs_meta_; }
  const Meta &GetRhsMeta() const;  // throws for single-input generators
  const Meta &GetOutputMeta() const { return output_meta_; }
  const flow::Attrs &GetAttrs() const { return attrs_; }

  // Equality over kind + metas (attribute-blind), used to share measured costs.
  size_t GetShapeHashCode() const;
  bool ShapeEquals(const KernelGenerator &other) const;
  // Equality over kind + metas + scalar/list attributes, used to dedupe generators.
  size_t GetHashCode() const;
  bool Equals(const KernelGenerator &other) const;

  // The four Yield* of the reference collapse to one: the family is the node's.
  std::shared_ptr<Kernel> Yield(const std::vector<size_t> &lhs_layout, const std::vector<size_t> &rhs_layout,
                                const std::vector<size_t> &output_layout);
  std::shared_ptr<Kernel> YieldSingleInputKernel(const std::vector<size_t> &input_layout,
                                                 const std::vector<size_t> &output_layout);
  std::shared_ptr<Kernel> YieldDoubleInputsKernel(const std::vector<size_t> &lhs_layout,
                                                  const std::vector<size_t> &rhs_layout,
                                                  const std::vector<size_t> &output_layout);

 private:
  flow::OpKind kind_;
  flow::Attrs attrs_;
  Meta lhs_meta_;
  std::optional<Meta> rhs_meta_;
  Meta output_meta_;
  bool has_buffer_;
  size_t buffer_size_;
  std::shared_ptr<Kernel> kernel_;  // created once, shared by every Yield
};

}  // namespace kernel
}  // namespace fluidml

#endif
