#include "structure/kernel/generator.h"

#include <functional>
#include <stdexcept>

#include "utils/utils.h"

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

namespace {
std::vector<size_t> LayoutOr(const std::vector<size_t> &layout, const Meta &meta) {
  return layout.empty() ? utils::GenDefaultLayout(meta.GetShape()) : layout;
}
void CheckHip(int rc, const char *what) {
  if (rc != 0) throw std::runtime_error(std::string(what) + ": " + fluidml_hip_error_string(rc));
}
}  // namespace

std::string KernelGenerator::GetContractionSignature(const std::vector<size_t> &lhs_layout,
                                                     const std::vector<size_t> &rhs_layout,
                                                     const std::vector<size_t> &output_layout) const {
  if (!IsContraction()) return std::string();
  // views at address 0: dense and 16-byte aligned, which is how the reference's generator fills its buffers too
  TensorView lhs(nullptr, lhs_meta_, LayoutOr(lhs_layout, lhs_meta_));
  TensorView rhs(nullptr, *rhs_meta_, LayoutOr(rhs_layout, *rhs_meta_));
  const TensorView out(nullptr, output_meta_, LayoutOr(output_layout, output_meta_));
  std::string epilogue = "standalone";
  if (kind_ == flow::OpKind::GemmConstantWeightsBias) {
    epilogue = std::string("gemm ta") + (attrs_.trans_a ? "1" : "0") + " tb" + (attrs_.trans_b ? "1" : "0");
  }
  return ContractionTable::Signature(KernelNameOf(kind_), lhs.t, rhs.t, out.t, 1, epilogue);
}

ContractPick KernelGenerator::MeasureStandalone(Kernel &kernel, const std::vector<size_t> &lhs_layout,
                                                const std::vector<size_t> &rhs_layout,
                                                const std::vector<size_t> &output_layout) const {
  // what the reference's generator does with FillBuffer'd host vectors and its Runner (generator/matmul.cpp:100-124)
  void *lhs_d = nullptr, *rhs_d = nullptr, *out_d = nullptr, *stream = nullptr, *start = nullptr, *stop = nullptr;
  ContractPick pick;
  auto release = [&]() {
    fluidml_hip_time_kernels(nullptr, nullptr);
    for (void *p : {lhs_d, rhs_d, out_d}) fluidml_hip_free(p);
    if (start) fluidml_hip_event_destroy(start);
    if (stop) fluidml_hip_event_destroy(stop);
    if (stream) fluidml_hip_stream_destroy(stream);
  };
  try {
    CheckHip(fluidml_hip_arena_create(lhs_meta_.GetSize(), &lhs_d), "tuning buffer");
    CheckHip(fluidml_hip_arena_create(rhs_meta_->GetSize(), &rhs_d), "tuning buffer");
    CheckHip(fluidml_hip_arena_create(output_meta_.GetSize(), &out_d), "tuning buffer");
    CheckHip(fluidml_hip_stream_create(&stream), "tuning stream");
    CheckHip(fluidml_hip_event_create(&start), "tuning event");
    CheckHip(fluidml_hip_event_create(&stop), "tuning event");
    kernel.Prepare();
    const TensorView lhs(lhs_d, lhs_meta_, LayoutOr(lhs_layout, lhs_meta_));
    const TensorView rhs(rhs_d, *rhs_meta_, LayoutOr(rhs_layout, *rhs_meta_));
    const TensorView out(out_d, output_meta_, LayoutOr(output_layout, output_meta_));
    auto &runnable = dynamic_cast<DoubleInputsWithoutBufferKernel &>(kernel);
    CheckHip(fluidml_hip_time_kernels(start, stop), "kernel timing on");
    auto launch = [&](uint32_t bits) {
      LaunchContext ctx;
      ctx.stream = stream;
      ctx.contract = bits;
      runnable.Run(ctx, lhs, rhs, out);
      return ctx.status;
    };
    auto elapsed = [&]() {
      double ns = 0;
      CheckHip(fluidml_hip_event_elapsed_ns(start, stop, &ns), "elapsed");
      return ns;
    };
    pick = ContractionTable::Measure(ContractionTable::Candidates(false), launch, elapsed, 3, kTuneMargin);
  } catch (...) {
    release();
    throw;
  }
  release();
  return pick;
}

std::shared_ptr<Kernel> KernelGenerator::Yield(const std::vector<size_t> &lhs_layout, const std::vector<size_t> &rhs_layout,
                                               const std::vector<size_t> &output_layout) {
  if (!IsContraction()) {
    if (!kernel_) kernel_ = MakeKernel(kind_, attrs_);
    return kernel_;
  }
  // one kernel per layout triple, carrying the tile configuration picked for it (reference generator/matmul.cpp:94-98:
  // `kernels_.find({lhs_layout, rhs_layout, output_layout})`)
  const LayoutTriple key{LayoutOr(lhs_layout, lhs_meta_), LayoutOr(rhs_layout, *rhs_meta_), LayoutOr(output_layout, output_meta_)};
  auto it = kernels_.find(key);
  if (it != kernels_.end()) return it->second;
  std::shared_ptr<Kernel> kernel = MakeKernel(kind_, attrs_);
  if (table_ != nullptr && table_->GetMode() != ContractionTable::Mode::Off) {
    const std::string signature = GetContractionSignature(lhs_layout, rhs_layout, output_layout);
    ContractPick pick;
    bool known = table_->Find(signature, &pick);
    if (!known && table_->GetMode() == ContractionTable::Mode::Measure && fluidml_hip_device_count() > 0) {
      pick = MeasureStandalone(*kernel, lhs_layout, rhs_layout, output_layout);
      table_->Put(signature, pick);
      known = true;
    }
    if (known) kernel->SetContractFlags(pick.Flags());
  }
  kernels_.insert({key, kernel});
  return kernel;
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
