#include "structure/kernel/generator.h"

#include <functional>
#include <stdexcept>

namespace fluidml {
namespace kernel {

namespace {
constexpr size_t kSeed = 0x9e3779b9;  // reference generator.cpp:6
inline void Mix(size_t &h, size_t v) { h ^= v + kSeed + (h << 6) + (h >> 2); }
void MixMeta(size_t &h, const Meta &m) {
  Mix(h, std::hash<Type>()(m.GetType()));
  for (int64_t d : m.GetShape()) Mix(h, std::hash<int64_t>()(d));
}
void MixInts(size_t &h, const std::vector<int64_t> &v) {
  for (int64_t x : v) Mix(h, std::hash<int64_t>()(x));
}
}  // namespace

KernelGenerator::KernelGenerator(const flow::Node &node)
    : kind_(node.GetKind()), attrs_(node.GetAttrs()), lhs_meta_(node.GetLhs()->GetMeta()),
      output_meta_(node.GetOutput()->GetMeta()), has_buffer_(node.HasBuffer()), buffer_size_(node.GetBufferSize()) {
  if (node.IsDoubleInputs()) rhs_meta_ = node.GetRhs()->GetMeta();
}

std::string KernelGenerator::GetKernelName() const { return KernelNameOf(kind_); }

const Meta &KernelGenerator::GetRhsMeta() const {
  if (!rhs_meta_) throw std::logic_error(GetKernelName() + " generator has a single input");
  return *rhs_meta_;
}

size_t KernelGenerator::GetShapeHashCode() const {
  size_t h = std::hash<int>()(static_cast<int>(kind_));
  MixMeta(h, lhs_meta_);
  if (rhs_meta_) MixMeta(h, *rhs_meta_);
  MixMeta(h, output_meta_);
  return h;
}

bool KernelGenerator::ShapeEquals(const KernelGenerator &o) const {
  if (kind_ != o.kind_ || lhs_meta_ != o.lhs_meta_ || output_meta_ != o.output_meta_) return false;
  if (static_cast<bool>(rhs_meta_) != static_cast<bool>(o.rhs_meta_)) return false;
  return !rhs_meta_ || *rhs_meta_ == *o.rhs_meta_;
}

size_t KernelGenerator::GetHashCode() const {
  size_t h = GetShapeHashCode();
  Mix(h, std::hash<double>()(attrs_.value));
  Mix(h, std::hash<double>()(attrs_.alpha));
  Mix(h, std::hash<double>()(attrs_.beta));
  Mix(h, std::hash<int64_t>()(attrs_.axis));
  Mix(h, std::hash<int64_t>()(attrs_.group));
  Mix(h, std::hash<int64_t>()(attrs_.index));
  MixInts(h, attrs_.axes);
  MixInts(h, attrs_.perm);
  MixInts(h, attrs_.kernel_shape);
  MixInts(h, attrs_.pads);
  MixInts(h, attrs_.strides);
  MixInts(h, attrs_.dilations);
  MixInts(h, attrs_.starts);
  MixInts(h, attrs_.steps);
  return h;
}

bool KernelGenerator::Equals(const KernelGenerator &o) const {
  const flow::Attrs &a = attrs_, &b = o.attrs_;
  auto same_tensor = [](const std::optional<Tensor> &x, const std::optional<Tensor> &y) {
    return static_cast<bool>(x) == static_cast<bool>(y) && (!x || *x == *y);
  };
  return ShapeEquals(o) && a.type == b.type && a.value == b.value && a.alpha == b.alpha && a.beta == b.beta &&
         a.extra == b.extra && a.trans_a == b.trans_a && a.trans_b == b.trans_b && a.axis == b.axis &&
         a.epsilon == b.epsilon && a.group == b.group && a.index == b.index && a.min == b.min && a.max == b.max &&
         a.keepdims == b.keepdims && a.axes == b.axes && a.dilations == b.dilations &&
         a.kernel_shape == b.kernel_shape && a.pads == b.pads && a.strides == b.strides && a.perm == b.perm &&
         a.starts == b.starts && a.ends == b.ends && a.steps == b.steps && a.pad_pairs == b.pad_pairs &&
         same_tensor(a.t0, b.t0) && same_tensor(a.t1, b.t1) && same_tensor(a.t2, b.t2);
}

std::shared_ptr<Kernel> KernelGenerator::Yield(const std::vector<size_t> &, const std::vector<size_t> &,
                                               const std::vector<size_t> &) {
  if (!kernel_) kernel_ = MakeKernel(kind_, attrs_);
  return kernel_;
}

std::shared_ptr<Kernel> KernelGenerator::YieldSingleInputKernel(const std::vector<size_t> &input_layout,
                                                                const std::vector<size_t> &output_layout) {
  if (!IsSingleInput()) throw std::logic_error(GetKernelName() + " generator has two inputs");
  return Yield(input_layout, {}, output_layout);
}

std::shared_ptr<Kernel> KernelGenerator::YieldDoubleInputsKernel(const std::vector<size_t> &lhs_layout,
                                                                 const std::vector<size_t> &rhs_layout,
                                                                 const std::vector<size_t> &output_layout) {
  if (IsSingleInput()) throw std::logic_error(GetKernelName() + " generator has a single input");
  return Yield(lhs_layout, rhs_layout, output_layout);
}

}  // namespace kernel
}  // namespace fluidml
