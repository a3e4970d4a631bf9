#include "structure/kernel/kernel.h"

#include <cstring>
#include <stdexcept>

#include "utils/utils.h"

namespace fluidml {
namespace kernel {

using flow::Attrs;
using flow::OpKind;

std::vector<std::vector<Axis>> GetAxesInAllOrders() {
  return {{i, j, k}, {i, k, j}, {j, i, k}, {j, k, i}, {k, i, j}, {k, j, i}};
}

void LaunchContext::Note(int code, const std::string &kernel_name) {
  if (code != 0 && status == 0) {
    status = code;
    failed = kernel_name;
  }
}

TensorView::TensorView() { std::memset(&t, 0, sizeof(t)); }

TensorView::TensorView(void *base, const Meta &meta, const std::vector<size_t> &layout) {
  std::memset(&t, 0, sizeof(t));
  const std::vector<int64_t> &shape = meta.GetShape();
  if (shape.size() > FL_MAX_RANK) throw std::invalid_argument("TensorView: rank above FL_MAX_RANK");
  const std::vector<int64_t> strides = utils::GenStrides(shape, layout);
  t.base = base;
  t.dtype = static_cast<int32_t>(meta.GetType());
  t.rank = static_cast<int32_t>(shape.size());
  for (size_t d = 0; d < shape.size(); ++d) {
    t.shape[d] = shape[d];
    t.strides[d] = strides[d];
  }
}

TensorView::TensorView(void *base, const Meta &meta) : TensorView(base, meta, utils::GenDefaultLayout(meta.GetShape())) {}

DeviceConstant::DeviceConstant(const Tensor &tensor) : tensor_(tensor) {}

DeviceConstant::~DeviceConstant() {
  if (device_ != nullptr) fluidml_hip_free(device_);
}

void DeviceConstant::Upload() {
  if (device_ != nullptr) return;
  const std::vector<uint8_t> bytes = tensor_.Pack(utils::GenDefaultLayout(tensor_.GetShape()));
  const int rc = fluidml_hip_upload_constant(bytes.data(), bytes.size(), &device_);
  if (rc != 0) throw std::runtime_error(std::string("uploading a kernel constant failed: ") + fluidml_hip_error_string(rc));
}

TensorView DeviceConstant::View() const {
  if (device_ == nullptr) throw std::logic_error("DeviceConstant::View before Upload");
  return TensorView(device_, tensor_.GetMeta());
}

std::string KernelNameOf(OpKind kind) { return std::string(flow::OpKindName(kind)) + "Kernel"; }

namespace {

class Base : virtual public Kernel {
 public:
  Base(OpKind kind, const Attrs &attrs) : kind_(kind), attrs_(attrs) {
    if (attrs.t0) c0_ = std::make_unique<DeviceConstant>(*attrs.t0);
    if (attrs.t1) c1_ = std::make_unique<DeviceConstant>(*attrs.t1);
    if (attrs.t2) c2_ = std::make_unique<DeviceConstant>(*attrs.t2);
    attrs_.t0.reset();  // the DeviceConstants own the data from here on
    attrs_.t1.reset();
    attrs_.t2.reset();
  }
  std::string GetKernelName() const override { return KernelNameOf(kind_); }
  void Prepare() override {
    for (DeviceConstant *c : {c0_.get(), c1_.get(), c2_.get()}) {
      if (c) c->Upload();
    }
  }
  const DeviceConstant *GetConstant(int i) const override {
    return i == 0 ? c0_.get() : i == 1 ? c1_.get() : i == 2 ? c2_.get() : nullptr;
  }
  size_t GetConstantBytes() const override {
    size_t n = 0;
    for (const DeviceConstant *c : {c0_.get(), c1_.get(), c2_.get()}) {
      if (c) n += c->GetSize();
    }
    return n;
  }
  void SetContractFlags(uint32_t bits) override { contract_ = bits; }
  uint32_t GetContractFlags() const override { return contract_; }

 protected:
  // fl_contract_flags of a launch: the bf16 switch of the context plus the tile configuration (the context's, else
  // this kernel's own)
  uint32_t ContractBits(const LaunchContext &ctx) const {
    return (ctx.bf16 ? static_cast<uint32_t>(FL_CONTRACT_BF16) : 0u) | (ctx.contract != 0 ? ctx.contract : contract_);
  }
  uint32_t contract_ = 0;
  const DeviceConstant &Const(const std::unique_ptr<DeviceConstant> &c, const char *what) const {
    if (!c) throw std::logic_error(GetKernelName() + ": missing constant " + what);
    return *c;
  }
  OpKind kind_;
  Attrs attrs_;
  std::unique_ptr<DeviceConstant> c0_, c1_, c2_;
};

int64_t NormAxis(int64_t axis, int32_t rank) { return axis < 0 ? axis + rank : axis; }

class SingleNoBuffer final : public SingleInputWithoutBufferKernel, public Base {
 public:
  using Base::Base;
  void Run(LaunchContext &ctx, const TensorView &input, const TensorView &output) const override {
    const fl_tensor *in = &input.t, *out = &output.t;
    void *s = ctx.stream;
    const Attrs &a = attrs_;
    int rc = FL_ERR_UNSUPPORTED;
    switch (kind_) {
      case OpKind::AddConstant: rc = fluidml_hip_add_constant(in, out, a.value, s); break;
      case OpKind::SubConstantLhs: rc = fluidml_hip_sub_constant_lhs(in, out, a.value, s); break;
      case OpKind::MulConstant: rc = fluidml_hip_mul_constant(in, out, a.value, s); break;
      case OpKind::DivConstantRhs: rc = fluidml_hip_div_constant_rhs(in, out, a.value, s); break;
      case OpKind::Pow: rc = fluidml_hip_pow(in, out, a.value, s); break;
      case OpKind::Erf: rc = fluidml_hip_erf(in, out, s); break;
      case OpKind::Relu: rc = fluidml_hip_relu(in, out, s); break;
      case OpKind::Clip: rc = fluidml_hip_clip(in, out, a.min, a.max, s); break;
      case OpKind::Tanh: rc = fluidml_hip_tanh(in, out, s); break;
      case OpKind::Sqrt: rc = fluidml_hip_sqrt(in, out, s); break;
      case OpKind::Neg: rc = fluidml_hip_neg(in, out, s); break;
      case OpKind::Not: rc = fluidml_hip_not(in, out, s); break;
      case OpKind::Cast: rc = fluidml_hip_cast(in, out, s); break;
      case OpKind::Equal: rc = fluidml_hip_equal(in, out, a.value, s); break;
      case OpKind::Dropout: rc = fluidml_hip_dropout(in, out, s); break;
      case OpKind::CumSum: rc = fluidml_hip_cum_sum(in, out, NormAxis(a.axis, in->rank), s); break;
      case OpKind::Flatten: rc = fluidml_hip_flatten(in, out, a.axis, s); break;
      case OpKind::Reshape: rc = fluidml_hip_reshape(in, out, s); break;
      case OpKind::Transpose:
        rc = fluidml_hip_transpose(in, out, a.perm.data(), static_cast<int32_t>(a.perm.size()), s);
        break;
      case OpKind::Squeeze:
        rc = fluidml_hip_squeeze(in, out, a.axes.data(), static_cast<int32_t>(a.axes.size()), s);
        break;
      case OpKind::Unsqueeze:
        rc = fluidml_hip_unsqueeze(in, out, a.axes.data(), static_cast<int32_t>(a.axes.size()), s);
        break;
      case OpKind::Slice: {
        // only start, axis and step are used; the extent is the output's (reference slice.cpp:28-40)
        std::vector<int64_t> starts(a.starts), axes(a.axes), steps(a.steps);
        for (size_t n = 0; n < axes.size(); ++n) {
          axes[n] = NormAxis(axes[n], in->rank);
          if (axes[n] >= 0 && axes[n] < in->rank && starts[n] < 0) starts[n] += in->shape[axes[n]];
        }
        rc = fluidml_hip_slice(in, out, starts.data(), axes.data(), steps.data(), static_cast<int32_t>(axes.size()), s);
        break;
      }
      case OpKind::Pad: {
        std::vector<int64_t> before;
        for (const auto &p : a.pad_pairs) before.push_back(std::get<0>(p));
        rc = fluidml_hip_pad(in, out, before.data(), static_cast<int32_t>(before.size()), ctx.flags, s);
        break;
      }
      case OpKind::ReduceMean: {
        if (!a.keepdims) break;  // unreachable in the reference (reduce_mean.cpp:56-62)
        std::vector<int64_t> axes(a.axes);
        for (int64_t &ax : axes) ax = NormAxis(ax, in->rank);
        rc = fluidml_hip_reduce_mean(in, out, axes.data(), static_cast<int32_t>(axes.size()), s);
        break;
      }
      case OpKind::MaxPoolWithoutPadding:
        rc = fluidml_hip_max_pool_without_padding(in, out, a.kernel_shape.data(), a.strides.data(),
                                                  static_cast<int32_t>(a.kernel_shape.size()), s);
        break;
      case OpKind::AveragePoolWithoutPadding:
        rc = fluidml_hip_average_pool_without_padding(in, out, a.kernel_shape.data(), a.strides.data(),
                                                      static_cast<int32_t>(a.kernel_shape.size()), s);
        break;
      case OpKind::GatherConstantIndexScalar:
        rc = fluidml_hip_gather_constant_index_scalar(in, out, a.axis, a.index, ctx.flags, s);
        break;
      case OpKind::GatherConstantIndicesTensor: {
        const TensorView idx = Const(c0_, "indices").View();
        rc = fluidml_hip_gather_constant_indices_tensor(in, &idx.t, out, NormAxis(a.axis, in->rank), s);
        break;
      }
      case OpKind::GatherConstantDataTensor: {
        const TensorView data = Const(c0_, "data").View();
        rc = fluidml_hip_gather_constant_data_tensor(in, &data.t, out, s);
        break;
      }
      case OpKind::GatherConstantDataTensorAddTensorLhsAddTensorLhs: {
        const TensorView data = Const(c0_, "data").View(), add0 = Const(c1_, "add0").View(),
                         add1 = Const(c2_, "add1").View();
        rc = fluidml_hip_gather_constant_data_tensor_add_tensor_lhs_add_tensor_lhs(in, &data.t, &add0.t, &add1.t, out, s);
        break;
      }
      case OpKind::WhereConstantCondConstantScalarY: {
        const TensorView cond = Const(c0_, "condition").View();
        rc = fluidml_hip_where_constant_cond_constant_scalar_y(&cond.t, in, out, a.value, s);
        break;
      }
      case OpKind::WhereConstantCondConstantTensorY: {
        const TensorView cond = Const(c0_, "condition").View(), y = Const(c1_, "y").View();
        rc = fluidml_hip_where_constant_cond_constant_tensor_y(&cond.t, in, &y.t, out, s);
        break;
      }
      case OpKind::AddDivErfAddMulMul: {
        const TensorView add0 = Const(c0_, "add0").View();
        rc = fluidml_hip_add_div_erf_add_mul_mul(in, &add0.t, out, a.alpha, a.beta, a.extra, s);
        break;
      }
      case OpKind::UnsqueezeSubLhsScalarMulRhsScalar:
        rc = fluidml_hip_unsqueeze_sub_lhs_scalar_mul_rhs_scalar(in, out, a.axes.data(),
                                                                 static_cast<int32_t>(a.axes.size()), a.alpha, a.beta, s);
        break;
      default: break;
    }
    ctx.Note(rc, GetKernelName());
  }
};

class SingleWithBuffer final : public SingleInputWithBufferKernel, public Base {
 public:
  using Base::Base;
  void Run(LaunchContext &ctx, const TensorView &input, const TensorView &output, const Buffer &buffer) const override {
    const fl_tensor *in = &input.t, *out = &output.t;
    int rc = FL_ERR_UNSUPPORTED;
    if (kind_ == OpKind::Softmax) {
      rc = fluidml_hip_softmax(in, out, buffer.ptr, buffer.bytes, NormAxis(attrs_.axis, in->rank), ctx.stream);
    } else if (kind_ == OpKind::LayerNormalizationConstantScaleBias) {
      const TensorView scale = Const(c0_, "scale").View(), bias = Const(c1_, "bias").View();
      rc = fluidml_hip_layer_normalization_constant_scale_bias(in, &scale.t, &bias.t, out, buffer.ptr, buffer.bytes,
                                                               attrs_.axis, attrs_.epsilon, ctx.flags, ctx.stream);
    }
    ctx.Note(rc, GetKernelName());
  }
};

class DoubleNoBuffer final : public DoubleInputsWithoutBufferKernel, public Base {
 public:
  using Base::Base;
  void Run(LaunchContext &ctx, const TensorView &lhs, const TensorView &rhs, const TensorView &output) const override {
    const fl_tensor *l = &lhs.t, *r = &rhs.t, *out = &output.t;
    void *s = ctx.stream;
    int rc = FL_ERR_UNSUPPORTED;
    switch (kind_) {
      case OpKind::AddCommon: rc = fluidml_hip_add_common(l, r, out, s); break;
      case OpKind::SubCommon: rc = fluidml_hip_sub_common(l, r, out, s); break;
      case OpKind::MulCommon: rc = fluidml_hip_mul_common(l, r, out, s); break;
      case OpKind::DivCommon: rc = fluidml_hip_div_common(l, r, out, s); break;
      case OpKind::Concat2: rc = fluidml_hip_concat2(l, r, out, NormAxis(attrs_.axis, out->rank), s); break;
      case OpKind::MatMul: {
        const uint32_t bits = ContractBits(ctx);
        // (the chain entry point with neither bias nor chain is the plain product, and takes the configuration)
        rc = bits == 0 ? fluidml_hip_matmul(l, r, out, s) : fluidml_hip_matmul_chain(l, r, nullptr, out, nullptr, bits, s);
        break;
      }
      case OpKind::GemmConstantWeightsBias: {
        const TensorView bias = Const(c0_, "bias").View();
        rc = fluidml_hip_gemm_constant_weights_bias(l, r, &bias.t, out, attrs_.alpha, attrs_.beta, attrs_.trans_a ? 1 : 0,
                                                    attrs_.trans_b ? 1 : 0, ctx.flags | (ContractBits(ctx) << FL_CONTRACT_SHIFT), s);
        break;
      }
      case OpKind::ConvWithoutPadding: {
        TensorView bias;
        if (c0_) bias = c0_->View();
        rc = fluidml_hip_conv_without_padding(l, r, c0_ ? &bias.t : nullptr, out, attrs_.strides.data(),
                                              attrs_.dilations.data(), attrs_.group, ctx.flags | (ContractBits(ctx) << FL_CONTRACT_SHIFT), s);
        break;
      }
      default: break;
    }
    ctx.Note(rc, GetKernelName());
  }
};

class DoubleWithBuffer final : public DoubleInputsWithBufferKernel, public Base {
 public:
  using Base::Base;
  void Run(LaunchContext &ctx, const TensorView &lhs, const TensorView &rhs, const TensorView &output,
           const Buffer &buffer) const override {
    int rc = FL_ERR_UNSUPPORTED;
    if (kind_ == OpKind::ConvWithPadding) {
      TensorView bias;
      if (c0_) bias = c0_->View();
      rc = fluidml_hip_conv_with_padding(&lhs.t, &rhs.t, c0_ ? &bias.t : nullptr, &output.t, buffer.ptr, buffer.bytes,
                                         attrs_.pads.data(), attrs_.strides.data(), attrs_.dilations.data(), attrs_.group,
                                         ctx.flags | (ContractBits(ctx) << FL_CONTRACT_SHIFT), ctx.stream);
    }
    ctx.Note(rc, GetKernelName());
  }
};

}  // namespace

std::unique_ptr<Kernel> MakeKernel(OpKind kind, const Attrs &attrs) {
  switch (kind) {
    case OpKind::Softmax:
    case OpKind::LayerNormalizationConstantScaleBias: return std::make_unique<SingleWithBuffer>(kind, attrs);
    case OpKind::ConvWithPadding: return std::make_unique<DoubleWithBuffer>(kind, attrs);
    case OpKind::AddCommon:
    case OpKind::SubCommon:
    case OpKind::MulCommon:
    case OpKind::DivCommon:
    case OpKind::Concat2:
    case OpKind::MatMul:
    case OpKind::GemmConstantWeightsBias:
    case OpKind::ConvWithoutPadding: return std::make_unique<DoubleNoBuffer>(kind, attrs);
    default: return std::make_unique<SingleNoBuffer>(kind, attrs);
  }
}

}  // namespace kernel
}  // namespace fluidml
