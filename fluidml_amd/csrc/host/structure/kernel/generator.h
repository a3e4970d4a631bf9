// Per-node kernel factories (reference include/structure/kernel/generator/generator.h:11-141).
// A generator knows a node's metas and attributes and yields the kernel for a
// given choice of operand layouts.  On this backend a kernel reads strides
// from its views at launch, so for most kinds the yielded object does not
// depend on the layouts.  MatMul and Gemm are the exception, as in the
// reference, whose generators time their kernel's variants for the layouts
// asked for and cache the fastest per layout triple
// (generator/matmul.cpp:88-131, gemm.cpp:106-151): here the variants are the
// tile configurations of the contraction kernel, looked up in -- or measured
// into -- the ContractionTable the generator was given.  The layouts also key
// the cost cache of the layout DP, and two generators that ShapeEquals share
// one cost-table entry exactly as in the reference (generator.cpp:8-42: same
// generator type and same metas, attributes ignored).
#ifndef FLUIDML_AMD_HOST_STRUCTURE_KERNEL_GENERATOR_H_
#define FLUIDML_AMD_HOST_STRUCTURE_KERNEL_GENERATOR_H_

#include <map>
#include <memory>
#include <string>
#include <tuple>
#include <vector>

#include "structure/flow/flow.h"
#include "structure/kernel/kernel.h"
#include "structure/kernel/tuner.h"

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

  // Where MatMul / Gemm generators look up (and, in its Measure mode, record) the tile configuration of the kernels
  // they yield.  Without a table every kernel launches with the library's rule.
  void SetContractionTable(std::shared_ptr<ContractionTable> table) { table_ = std::move(table); }
  // The problem signature of this node's contraction under the given layouts, operands dense and aligned
  // (the key of the ContractionTable); empty for kinds other than MatMul / Gemm.
  std::string GetContractionSignature(const std::vector<size_t> &lhs_layout, const std::vector<size_t> &rhs_layout,
                                      const std::vector<size_t> &output_layout) const;

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
  using LayoutTriple = std::tuple<std::vector<size_t>, std::vector<size_t>, std::vector<size_t>>;
  bool IsContraction() const { return kind_ == flow::OpKind::MatMul || kind_ == flow::OpKind::GemmConstantWeightsBias; }
  // times the admissible tile configurations of the standalone kernel on zero-filled buffers of its own
  ContractPick MeasureStandalone(Kernel &kernel, const std::vector<size_t> &lhs_layout, const std::vector<size_t> &rhs_layout,
                                 const std::vector<size_t> &output_layout) const;
  std::shared_ptr<Kernel> kernel_;  // kinds other than MatMul / Gemm: created once, shared by every Yield
  std::map<LayoutTriple, std::shared_ptr<Kernel>> kernels_;  // MatMul / Gemm: one per layout triple, with its pick
  std::shared_ptr<ContractionTable> table_;
};

}  // namespace kernel
}  // namespace fluidml

#endif
