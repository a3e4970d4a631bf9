#include "worker/builder.h"

#include <stdexcept>
#include <unordered_set>

#include "utils/utils.h"
#include "worker/launcher.h"
#include "worker/utils.h"

namespace fluidml {
namespace worker {
namespace {

double NumelOf(const Meta &m) { return static_cast<double>(m.GetElementsNum()); }

// Algorithmic bytes and flops of one node: every operand counted once at its
// own size, broadcast operands at their (small) size, scratch excluded;
// flops only for the contractions.
void AccountWork(const flow::Node &node, Step *step) {
  using flow::OpKind;
  const flow::Attrs &a = node.GetAttrs();
  const Meta &in = node.GetLhs()->GetMeta(), &out = node.GetOutput()->GetMeta();
  double bytes = static_cast<double>(out.GetSize());
  double flops = 0;
  auto tensor_bytes = [](const std::optional<Tensor> &t) { return t ? static_cast<double>(t->GetMeta().GetSize()) : 0.0; };
  switch (node.GetKind()) {
    case OpKind::GatherConstantDataTensor:
    case OpKind::GatherConstantDataTensorAddTensorLhsAddTensorLhs:
      // the rows that are read, not the whole table
      bytes += static_cast<double>(in.GetSize()) + static_cast<double>(out.GetSize()) + tensor_bytes(a.t1) + tensor_bytes(a.t2);
      break;
    case OpKind::GatherConstantIndexScalar:
    case OpKind::GatherConstantIndicesTensor:
    case OpKind::Slice:
      bytes += static_cast<double>(out.GetSize()) + tensor_bytes(a.t0);  // only the gathered part of the input moves
      break;
    case OpKind::MatMul: {
      const Meta &rhs = node.GetRhs()->GetMeta();
      bytes += static_cast<double>(in.GetSize()) + static_cast<double>(rhs.GetSize());
      flops = 2.0 * NumelOf(out) * static_cast<double>(in.GetShape().back());
      break;
    }
    case OpKind::GemmConstantWeightsBias: {
      const Meta &rhs = node.GetRhs()->GetMeta();
      bytes += static_cast<double>(in.GetSize()) + static_cast<double>(rhs.GetSize()) + tensor_bytes(a.t0);
      const double k = static_cast<double>(a.trans_a ? in.GetShape()[0] : in.GetShape()[1]);
      flops = 2.0 * NumelOf(out) * k;
      break;
    }
    case OpKind::ConvWithPadding:
    case OpKind::ConvWithoutPadding: {
      const Meta &w = node.GetRhs()->GetMeta();
      bytes += static_cast<double>(in.GetSize()) + static_cast<double>(w.GetSize()) + tensor_bytes(a.t0);
      double taps = 1;
      for (size_t d = 1; d < w.GetShape().size(); ++d) taps *= static_cast<double>(w.GetShape()[d]);  // C/g * prod(k)
      flops = 2.0 * NumelOf(out) * taps + (a.t0 ? NumelOf(out) : 0.0);
      break;
    }
    default:
      bytes += static_cast<double>(in.GetSize()) + tensor_bytes(a.t0) + tensor_bytes(a.t1) + tensor_bytes(a.t2);
      if (node.IsDoubleInputs()) bytes += static_cast<double>(node.GetRhs()->GetMeta().GetSize());
  }
  step->bytes = bytes;
  step->flops = flops;
}

class GeneralBuilderImpl : public GeneralBuilder {
 public:
  GeneralBuilderImpl(std::string &&function_name, context::Context &&context, bool from_generators)
      : function_name_(std::move(function_name)), context_(std::move(context)), from_generators_(from_generators) {}

  void Run(const flow::Sequence &sequence, const memory::Index &index) override {
    const size_t arena_bytes = index.GetMaximum();
    std::string name = function_name_;
    auto plan = std::make_unique<LaunchPlan>(std::move(name), arena_bytes);
    name = function_name_;
    context::FuncAttr func_attr(std::move(name), arena_bytes);

    // regions that no Memory edge touches were planned with an empty lifetime:
    // they must not be written inside the arena
    std::unordered_set<std::string> linked;
    for (const std::shared_ptr<flow::Edge> &edge : sequence.GetEdges()) {
      if (edge->IsMemory()) linked.insert(edge->GetName());
    }
    for (const std::shared_ptr<flow::Region> &region : sequence.GetRegions()) {
      switch (region->GetKind()) {
        case flow::Region::Kind::Input:
        case flow::Region::Kind::Output: {
          const bool is_input = region->GetKind() == flow::Region::Kind::Input;
          std::string arg_name = region->GetName();
          func_attr.PutArgument(context::ArgumentAttr(
              is_input ? context::ArgumentAttr::Type::Input : context::ArgumentAttr::Type::Output, std::move(arg_name),
              Meta(region->GetMeta())));
          plan->AddArgument(Argument{is_input ? Argument::Type::Input : Argument::Type::Output, region->GetName(),
                                     region->GetMeta()});
          break;
        }
        case flow::Region::Kind::Constant:
          plan->AddConstant(region->GetName(), region->GetTensor(), region->GetLayout());
          break;
        case flow::Region::Kind::Inner:
          if (!linked.count(region->GetName())) plan->AddPrivate(region->GetName(), region->GetMeta().GetSize());
          break;
      }
    }
    auto operand_of = [&](const std::shared_ptr<flow::Region> &region) {
      Operand op;
      op.name = region->GetName();
      op.meta = region->GetMeta();
      op.layout = region->GetLayout();
      switch (region->GetKind()) {
        case flow::Region::Kind::Inner:
          if (linked.count(op.name)) {
            op.space = Operand::Space::Arena;
            op.offset = index.Get(op.name);
          } else {
            op.space = Operand::Space::Private;
          }
          break;
        case flow::Region::Kind::Constant: op.space = Operand::Space::Constant; break;
        default:
          // interface tensors keep dense row-major storage whatever layout the
          // DP wrote into the region (reference builder.cpp:193)
          op.space = Operand::Space::Interface;
          op.layout = utils::GenDefaultLayout(op.meta.GetShape());
      }
      return op;
    };
    for (const std::shared_ptr<flow::Node> &node : sequence.GetNodes()) {
      Step step;
      step.node = node;
      if (from_generators_) {
        std::unique_ptr<kernel::KernelGenerator> generator = SelectKernelGenerator(node.get());
        generator->SetContractionTable(context_->contraction_table);
        step.kernel = generator->Yield(node->GetLhs()->GetLayout(),
                                       node->IsDoubleInputs() ? node->GetRhs()->GetLayout() : std::vector<size_t>{},
                                       node->GetOutput()->GetLayout());
      } else {
        step.kernel = SelectKernel(node.get());
      }
      step.in0 = operand_of(node->GetLhs());
      if (node->IsDoubleInputs()) step.in1 = operand_of(node->GetRhs());
      step.out = operand_of(node->GetOutput());
      const size_t scratch = node->GetBufferSize();
      step.has_buffer = node->HasBuffer();
      if (scratch > 0) {
        step.buffer_offset = index.Get(node->GetName());
        step.buffer_bytes = scratch;
      }
      AccountWork(*node, &step);
      plan->AddStep(std::move(step));
    }
    plan->SetFlags(context_->ref_flags);
    plan->SetUseGraph(context_->use_graph);
    plan->SetFuse(context_->fuse);
    plan->SetBf16(context_->bf16);
    if (context_->branch_min_us >= 0) plan->SetBranchMinUs(context_->branch_min_us);
    plan->SetBranchCheck(context_->branch_check);
    plan->SetBranchDecision(context_->branch_decision);
    plan->SetContractionTable(context_->contraction_table);
    context_->SetModule(std::move(plan));
    context_->SetFuncAttr(std::move(func_attr));
  }

 private:
  std::string function_name_;
  context::Context context_;
  bool from_generators_;
};

class KernelBuilderImpl : public KernelBuilder {
 public:
  KernelBuilderImpl(std::string &&function_name, context::Context &&context)
      : function_name_(std::move(function_name)), context_(std::move(context)) {}

  void RunOnSingleInputWithoutBuffer(std::shared_ptr<kernel::SingleInputWithoutBufferKernel> kernel, const Meta &input_meta,
                                     const std::vector<size_t> &input_layout, const Meta &output_meta,
                                     const std::vector<size_t> &output_layout) override {
    Build(std::move(kernel), {{kInputKey, input_meta, input_layout}}, {kOutputKey, output_meta, output_layout}, false, 0);
  }
  void RunOnSingleInputWithBuffer(std::shared_ptr<kernel::SingleInputWithBufferKernel> kernel, const Meta &input_meta,
                                  const std::vector<size_t> &input_layout, const Meta &output_meta,
                                  const std::vector<size_t> &output_layout, size_t buffer_size) override {
    Build(std::move(kernel), {{kInputKey, input_meta, input_layout}}, {kOutputKey, output_meta, output_layout}, true, buffer_size);
  }
  void RunOnDoubleInputsWithoutBuffer(std::shared_ptr<kernel::DoubleInputsWithoutBufferKernel> kernel, const Meta &lhs_meta,
                                      const std::vector<size_t> &lhs_layout, const Meta &rhs_meta,
                                      const std::vector<size_t> &rhs_layout, const Meta &output_meta,
                                      const std::vector<size_t> &output_layout) override {
    Build(std::move(kernel), {{kLhsKey, lhs_meta, lhs_layout}, {kRhsKey, rhs_meta, rhs_layout}},
          {kOutputKey, output_meta, output_layout}, false, 0);
  }
  void RunOnDoubleInputsWithBuffer(std::shared_ptr<kernel::DoubleInputsWithBufferKernel> kernel, const Meta &lhs_meta,
                                   const std::vector<size_t> &lhs_layout, const Meta &rhs_meta,
                                   const std::vector<size_t> &rhs_layout, const Meta &output_meta,
                                   const std::vector<size_t> &output_layout, size_t buffer_size) override {
    Build(std::move(kernel), {{kLhsKey, lhs_meta, lhs_layout}, {kRhsKey, rhs_meta, rhs_layout}},
          {kOutputKey, output_meta, output_layout}, true, buffer_size);
  }

 private:
  struct Arg {
    const char *key;
    Meta meta;
    std::vector<size_t> layout;
  };
  // A one-step plan: operands are interface tensors stored with the requested
  // layouts, scratch is the whole arena (reference builder.cpp:637-960).
  void Build(std::shared_ptr<kernel::Kernel> kernel, std::vector<Arg> inputs, Arg output, bool has_buffer,
             size_t buffer_size) {
    std::string name = function_name_;
    auto plan = std::make_unique<LaunchPlan>(std::move(name), buffer_size);
    name = function_name_;
    context::FuncAttr func_attr(std::move(name), buffer_size);
    auto operand = [&](const Arg &a, bool is_input) {
      std::string arg_name = a.key;
      func_attr.PutArgument(context::ArgumentAttr(is_input ? context::ArgumentAttr::Type::Input : context::ArgumentAttr::Type::Output,
                                                  std::move(arg_name), Meta(a.meta)));
      plan->AddArgument(Argument{is_input ? Argument::Type::Input : Argument::Type::Output, a.key, a.meta});
      Operand op;
      op.space = Operand::Space::Interface;
      op.name = a.key;
      op.meta = a.meta;
      op.layout = a.layout.empty() ? utils::GenDefaultLayout(a.meta.GetShape()) : a.layout;
      return op;
    };
    // a throw-away node gives the step its arity; its regions mirror the args
    auto region = [](const Arg &a, flow::Region::Kind kind) {
      return std::make_shared<flow::Region>(kind, std::string(a.key), Meta(a.meta));
    };
    Step step;
    step.kernel = std::move(kernel);
    step.in0 = operand(inputs[0], true);
    if (inputs.size() == 2) {
      step.in1 = operand(inputs[1], true);
      step.node = std::make_shared<flow::Node>(function_name_ + "-node", flow::OpKind::MatMul,
                                               region(inputs[0], flow::Region::Kind::Input),
                                               region(inputs[1], flow::Region::Kind::Input),
                                               region(output, flow::Region::Kind::Output));
    } else {
      step.node = std::make_shared<flow::Node>(function_name_ + "-node", flow::OpKind::Dropout,
                                               region(inputs[0], flow::Region::Kind::Input),
                                               region(output, flow::Region::Kind::Output));
    }
    step.out = operand(output, false);
    step.has_buffer = has_buffer;
    step.buffer_offset = 0;
    step.buffer_bytes = buffer_size;
    plan->AddStep(std::move(step));
    plan->SetFlags(context_->ref_flags);
    plan->SetUseGraph(false);
    plan->SetFuse(false);
    context_->SetModule(std::move(plan));
    context_->SetFuncAttr(std::move(func_attr));
  }

  std::string function_name_;
  context::Context context_;
};

}  // namespace

std::unique_ptr<GeneralBuilder> GeneralBuilder::MakePlain(std::string &&function_name, context::Context &&context) {
  return std::make_unique<GeneralBuilderImpl>(std::move(function_name), std::move(context), false);
}

std::unique_ptr<GeneralBuilder> GeneralBuilder::MakeDynamicProgramming(std::string &&function_name, context::Context &&context) {
  return std::make_unique<GeneralBuilderImpl>(std::move(function_name), std::move(context), true);
}

std::unique_ptr<KernelBuilder> KernelBuilder::Make(std::string &&function_name, context::Context &&context) {
  return std::make_unique<KernelBuilderImpl>(std::move(function_name), std::move(context));
}

}  // namespace worker
}  // namespace fluidml
