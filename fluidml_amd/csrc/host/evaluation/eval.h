// Time-cost evaluation feeding the layout DP (reference include/evaluation/eval.h,
// src/evaluation/eval.cpp, src/worker/evaluator.cpp).
//
// The reference JIT-compiles a one-kernel module per layout tuple and times
// one cold run on the host clock.  Here the same question -- "what does this
// kernel cost with these operand layouts" -- is answered by timing launches of
// the gfx950 kernel between hipEvents on warm buffers (minimum of a few runs),
// by the constant 1 (the reference's DP_DEBUG build), or from a cost table
// saved by an earlier compile, so a layout choice can be replayed exactly.
#ifndef FLUIDML_AMD_HOST_EVALUATION_EVAL_H_
#define FLUIDML_AMD_HOST_EVALUATION_EVAL_H_

#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "structure/context/context.h"
#include "structure/kernel/generator.h"

namespace fluidml {
namespace evaluation {

using Layout = std::vector<size_t>;
// (lhs | input, rhs | empty, output)
using LayoutKey = std::vector<Layout>;

class KernelEval;

// Source of costs; one per Context.
class CostModel {
 public:
  virtual ~CostModel() = default;
  // nanoseconds (or the constant 1) for `eval`'s kernel under `key`
  virtual size_t Cost(KernelEval &eval, const LayoutKey &key) = 0;
  // What the last Cost() call measured, in nanoseconds, before any margin the model adds for the DP's comparison;
  // 0 when that cost was not a measurement (a constant, an estimate for a candidate left untimed).
  double LastMeasuredNs() const { return last_measured_ns_; }
  virtual bool IsMeasuring() const { return false; }  // true: costs come from timing kernels on the device

 protected:
  double last_measured_ns_ = 0;

 public:
  static std::shared_ptr<CostModel> Make(context::Context &context);
  static std::shared_ptr<CostModel> MakeConstant();
  static std::shared_ptr<CostModel> MakeMeasured(uint32_t ref_flags,
                                                 std::shared_ptr<kernel::ContractionTable> table = nullptr);
  // `json_text` is a report written by DynamicProgrammingTable::ToJson (bare or
  // wrapped as {"dp_table": ..., "plan": ...}); a lookup that misses throws
  static std::shared_ptr<CostModel> MakeFromTable(const std::string &json_text);
};

// Costs of one kernel shape, cached per layout tuple (reference eval.h:19-230).
class KernelEval {
 public:
  KernelEval(std::shared_ptr<kernel::KernelGenerator> generator, std::shared_ptr<CostModel> model);
  const kernel::KernelGenerator &GetKernelGenerator() const { return *generator_; }
  kernel::KernelGenerator &GetKernelGenerator() { return *generator_; }
  bool IsSingleInput() const { return generator_->IsSingleInput(); }
  size_t GetTimeCost(const Layout &input_layout, const Layout &output_layout);
  size_t GetTimeCost(const Layout &lhs_layout, const Layout &rhs_layout, const Layout &output_layout);
  size_t GetShortestTimeCost();  // minimum over every layout tuple
  // [{"input_shape"|"lhs_shape"+"rhs_shape", "output_shape", "*_layout"..., "time_cost"[, "dp_cost", "measured"]}, ...]
  // "time_cost" is the measured kernel time wherever there is one (what the reference's table and its analyzer
  // mean by it); "dp_cost", present where it differs, is what the DP compared (the measurement plus the margin
  // for non-default layouts, or the estimate of a candidate that was not timed: "measured": false).
  std::string ToJson() const;
  const std::map<LayoutKey, size_t> &GetTimeCosts() const { return time_costs_; }

 private:
  size_t Lookup(LayoutKey &&key);
  std::shared_ptr<kernel::KernelGenerator> generator_;
  std::shared_ptr<CostModel> model_;
  std::map<LayoutKey, size_t> time_costs_;
  std::map<LayoutKey, double> measured_ns_;  // per tuple: the raw measurement behind the cost (0: none)
};

}  // namespace evaluation

namespace worker {

// Node name -> KernelEval, with evals shared between nodes whose generators
// ShapeEquals (reference include/worker/evaluator.h, evaluator.cpp:12-31, 78-87).
class Evaluator {
 public:
  void RegisterEval(std::string &&name, std::shared_ptr<evaluation::KernelEval> &&eval);
  evaluation::KernelEval &GetEval(const std::string &name);
  evaluation::KernelEval &GetSingleInputEval(const std::string &name);
  evaluation::KernelEval &GetDoubleInputsEval(const std::string &name);
  // {<KernelName>: [entries of every distinct eval of that kernel...]}
  std::string ToJson() const;
  static std::shared_ptr<Evaluator> Make();

 private:
  std::vector<std::shared_ptr<evaluation::KernelEval>> evals_;  // distinct, registration order
  std::unordered_multimap<size_t, size_t> by_shape_hash_;       // shape hash -> index into evals_
  std::unordered_map<std::string, std::shared_ptr<evaluation::KernelEval>> by_name_;
};

}  // namespace worker
}  // namespace fluidml

#endif
