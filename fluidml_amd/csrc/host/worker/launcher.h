// The compiled artefact of this backend: an ordered list of kernel launches
// over one HBM arena.  It stands where the reference keeps an MLIR module plus
// a JIT engine (src/structure/context/context.cpp:152-166): GeneralBuilder
// fills it (reference builder.cpp:149-394 lays memref views over the arena
// argument), Lower validates it, Runner materialises it on the device and
// replays it.
#ifndef FLUIDML_AMD_HOST_WORKER_LAUNCHER_H_
#define FLUIDML_AMD_HOST_WORKER_LAUNCHER_H_

#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "structure/flow/flow.h"
#include "structure/kernel/kernel.h"
#include "structure/kernel/tuner.h"

namespace fluidml {
namespace worker {

// Where an operand of a step lives.
struct Operand {
  enum class Space {
    Arena,      // inner region: arena base + offset from the memory plan
    Interface,  // graph input/output: device staging buffer (GeneralBuilder gives it the identity layout)
    Constant,   // constant region: its own HBM allocation, region layout applied
    Private     // inner region no Memory edge uses: its own HBM allocation
  };
  Space space = Space::Arena;
  std::string name;
  size_t offset = 0;  // Arena; Private inside a shared buffer
  std::string pool;   // Private only: the shared buffer the tensor lives in at `offset` (empty: an allocation of its own)
  Meta meta{Type::kUnknown, std::vector<int64_t>{}};
  std::vector<size_t> layout;
  // A tensor that is not materialised but read through the bytes of another one (the output of an elided
  // Slice / Transpose / Squeeze / Unsqueeze / Reshape): `space`, `name` and `offset` are then the source's,
  // `meta` stays the view's own, and the view's logical element (i0, i1, ...) lives `view_offset +
  // sum(i_d * view_strides[d])` elements into the source, whose whole extent is `source_bytes`.
  bool viewed = false;
  int64_t view_offset = 0;
  std::vector<int64_t> view_strides;
  size_t source_bytes = 0;
  // bytes the operand may touch (its own, or its source's when it is a view)
  size_t Extent() const { return viewed ? source_bytes : meta.GetSize(); }
};

struct Step {
  std::shared_ptr<flow::Node> node;
  std::shared_ptr<kernel::Kernel> kernel;
  Operand in0, in1, out;  // in1 unused for single-input nodes
  bool has_buffer = false;
  size_t buffer_offset = 0, buffer_bytes = 0;
  // algorithmic work of the step: bytes = unique operand bytes + output bytes
  // (scratch excluded), flops = 2*MACs for contractions, 0 otherwise
  double bytes = 0, flops = 0;
};

// One launch of the replayed schedule: a single step, or a chain of steps whose
// intermediate tensors each have exactly one reader inside the chain.  A chain
// is issued at the position of its last member, reads only what enters the
// chain from outside, and writes only the last member's output; the elided
// intermediates keep their slots in the memory plan but are never touched.
struct Launch {
  enum class Kind {
    Step,              // members = {i}
    MatMulChain,       // MatMul [-> AddCommon(rank-1 constant bias)] [-> elementwise chain]
                       // [-> AddCommon(tensor) [-> AddCommon(tensor)]]
    GemmChain,         // GemmConstantWeightsBias -> elementwise chain
    ConvChain,         // [MulCommon(x, factor per channel) ->] Conv{With,Without}Padding -> elementwise chain
                       // [-> AddCommon(tensor of the output's shape)] | [+ ReduceMean over the spatial dims, second output]
    ConvPair,          // two pointwise convolutions on one-pixel tensors, each with its elementwise chain
                       // (squeeze-and-excitation): a = input, b = weights of `owner`, c = weights of `owner2`,
                       // `chain` follows the first, `chain2` the second
    SoftmaxMatVec,     // Softmax over <= 16 logits [B, K, 1] -> MatMul [B, M, K] x [B, K, 1] [-> Reshape views]:
                       // a = the matrix, b = the logits, view_strides as for MatMulChain
    MatMulGroup,       // up to four MatMulChains that share the left operand and all extents, one launch
    ElementwiseChain,  // two or more elementwise steps on one tensor
    MulAdd,            // MulCommon -> AddCommon: a * b + c
    AddAdd,            // AddCommon -> AddCommon: (a + b) + c
    GatherAdd,         // GatherConstantDataTensor -> AddCommon [-> AddCommon]: data[a] + b [+ c] (has_c), the
                       // table is the constant of `owner`
    Rotary,            // rotary position embedding (Slice, Neg, Concat2, MulCommon, AddCommon, Concat2 [, Transpose]):
                       // a = x, b = cosine table, c = sine table, axis = number of rotated values, perm = the
                       // folded Transpose (empty: none)
    RotaryPair,        // two Rotary launches next to each other with the same tables (queries and keys of a layer) as
                       // one launch: `group` holds the two, members = union of theirs, both outputs are written
    DivAddSoftmax,     // DivConstantRhs -> AddCommon(mask) -> Softmax
    Attention,         // MatMul -> Div|Mul constant [-> AddCommon(mask)] [-> Where(cond, x, scalar)] -> Softmax -> MatMul
    AddLayerNorm,      // AddCommon -> LayerNormalizationConstantScaleBias
    GatherAddLayerNorm,  // [GatherConstantDataTensor ->] GatherConstantDataTensor -> AddCommon -> AddCommon ->
                         // LayerNormalizationConstantScaleBias (last dim): a = indices into the table of `owner`,
                         // b = the first addend, or with has_gate the indices into the table of `owner2`, c = the
                         // second addend, `norm_owner` = the LayerNormalization step, s0 = epsilon
    GatherStats,       // GatherConstantDataTensor whose result feeds LayerNormalizations that are not run: a = indices
                       // into the table of `owner`; leaves the partial row statistics in `norm_stats_out`
    ReshapeTranspose,  // Reshape -> Transpose, one strided copy
    TransposeReshape,  // Transpose -> Reshape, one strided copy
    PadViewCopy,       // Pad -> steps that only re-address its result (Gather of sliding windows, Slice, Transpose,
                       // Reshape): a = the Pad's input, `view_offset` / `view_strides` = the last step's output inside
                       // the padded tensor (never written), out = the last step's output
    View,              // a Slice / Transpose / Squeeze / Unsqueeze / Reshape that is not run: its readers address
                       // the source through strides (members = {i}, out = the source operand seen as the view)
    Placed,            // a Concat2 that is not run: the launches producing its inputs wrote them into its output
    CopyInto           // a Concat2 one input of which was written in place by its producer: copies the other (a)
                       // into its part of the output (out, a view of the Concat2's output)
  };
  Kind kind = Kind::Step;
  std::vector<size_t> members;  // indices into the step list, ascending
  Operand a, b, c, d, e, out;   // external operands, role by kind (see fusion.cpp)
  // ConvChain that also delivers the ReduceMean over the spatial dims of its result (the ReduceMean is the last
  // member, `out` the tensor it reads, which is written too)
  Operand out2;
  bool has_out2 = false;
  double s0 = 0, s1 = 0, s2 = 0;
  int64_t axis = 0;
  std::vector<int64_t> perm;
  bool has_c = false;     // MatMulChain: a bias operand is present
  // ConvChain: c = a per-channel factor of the input (the MulCommon in front of the convolution is a member),
  // d = a tensor of the output's shape added after the chain (the AddCommon behind it is a member)
  // MatMulChain: d [and e] = tensors of the output's shape added after the chain, in this order (the AddCommon
  // steps are members): has_skip [and has_skip2]
  bool has_gate = false, has_skip = false, has_skip2 = false;
  // ConvChain: the tensor in `d` multiplies the value instead of being added to it (a MulCommon behind the convolution)
  bool skip_is_factor = false;
  // Attention: a = queries, b = keys (transposed), c = values, d = additive mask (has_mask), the Where step
  // `owner` holds the condition (has_cond) and s1 its fill value; s0 scales the scores, dividing if `divisor`
  bool has_mask = false, has_cond = false, divisor = false;
  // Step: the step's operands a, b, out replace the plan's when an input became a view of another tensor or the
  // output is written straight into a Concat2's output (rewired)
  bool rewired = false;
  // MatMulChain followed by Reshape/Transpose steps that only re-address the result: element strides of the
  // contraction's logical output dims inside `out` (empty: `out` is the contraction's own output tensor),
  // and the optional split of the last dim (see fluidml_hip_matmul_chain_view)
  std::vector<int64_t> view_strides;
  int64_t n_inner = 0, stride_outer = 0;
  int64_t view_offset = 0;  // PadViewCopy
  // MatMulGroup: the grouped chains (members = union of theirs; every chain's `out` is written)
  std::vector<Launch> group;
  size_t position = 0;  // MatMulGroup: step index where the launch is issued (one of the members)
  fl_ew_program chain{};  // elementwise steps applied to the value (n == 0: none)
  fl_ew_program chain2{};  // ConvPair: the steps after the second convolution
  size_t owner = 0;  // member whose kernel owns constants / attributes the launch needs (LayerNorm, Gemm, Conv)
  size_t owner2 = 0;  // ConvPair: the second convolution
  double bytes = 0, flops = 0;
  // A LayerNormalization that is not run: the contraction in front of it stores the tensor it would have normalised
  // (in the LayerNormalization's output buffer) together with partial row statistics, and its readers normalise on
  // the fly (fluidml_hip_matmul_chain_group_norm).  MatMulChain / MatMulGroup:
  //   norm_mode 1: `a` is such a tensor (the launch multiplies LayerNorm(a)); 2: the addend `d` is.  `norm_owner` is
  //   the LayerNormalization step whose scale, shift and epsilon apply, `norm_stats` the private buffer with the row
  //   statistics of the deferred operand.
  //   norm_stats_out (non-empty): the launch absorbed the LayerNormalization step behind it and leaves the partial
  //   row statistics of its result in that private buffer; `out` is the LayerNormalization's output tensor.
  int norm_mode = 0;
  size_t norm_owner = 0;
  std::string norm_stats, norm_stats_out;
  // MatMulChain / MatMulGroup / GemmChain, and a Step whose node is a MatMul or Gemm: the tile configuration the
  // launch runs with (FL_CONTRACT_TILE / FL_CONTRACT_SPLITS bits; 0 = the library's rule), set from the plan's
  // ContractionTable once the plan is on the device
  uint32_t contract = 0;
};
const char *LaunchKindName(Launch::Kind kind);
// Groups `steps` into launches.  With `fuse` false every step is its own launch.
// A chain is only formed when no step between its first and last member writes
// bytes that alias one of the chain's external inputs (arena intervals from the
// memory plan), so that issuing the reads late is safe.
std::vector<Launch> BuildSchedule(const std::vector<Step> &steps, bool fuse);

struct Argument {
  enum class Type { Input, Output };
  Type type;
  std::string name;
  Meta meta;
};

struct StepTime {
  std::string node, kernel;
  double ns = 0, bytes = 0, flops = 0;
};

class LaunchPlan {
 public:
  LaunchPlan(std::string &&name, size_t arena_bytes);
  ~LaunchPlan();
  LaunchPlan(const LaunchPlan &) = delete;

  // ---- filled by the builders (host only, no device needed) ----
  void AddArgument(Argument &&arg);
  void AddConstant(const std::string &name, const Tensor &tensor, const std::vector<size_t> &layout);
  void AddPrivate(const std::string &name, size_t bytes);
  void AddStep(Step &&step);

  const std::string &GetName() const { return name_; }
  size_t GetArenaBytes() const { return arena_bytes_; }
  size_t GetConstantBytes() const;   // constant regions + constants kernels own
  size_t GetInterfaceBytes() const;  // device staging of graph inputs and outputs
  size_t GetPrivateBytes() const;    // tensors outside the arena: regions no Memory edge uses, outputs of side branches
  size_t GetPeakDeviceBytes() const { return arena_bytes_ + GetConstantBytes() + GetInterfaceBytes() + GetPrivateBytes(); }
  const std::vector<Step> &GetSteps() const { return steps_; }
  // the launches actually replayed (steps grouped into chains when fusion is on)
  const std::vector<Launch> &GetSchedule() const;
  const std::vector<Argument> &GetArguments() const { return arguments_; }
  // Every arena operand and scratch buffer lies inside [0, arena_bytes); every
  // named constant / interface / private operand exists. Throws std::logic_error otherwise.
  void Validate() const;
  // Human-readable listing (what the `mlir` / `llvm` sinks of Executor::Compile receive).
  std::string ToText() const;

  // ---- device side ----
  // Allocates the arena, uploads constants, allocates interface staging and
  // prepares kernels. Idempotent. Throws std::runtime_error on HIP errors.
  void Materialize();
  bool IsMaterialized() const { return arena_ != nullptr; }
  // Materialize(), then everything the first run would decide by timing (the side branches), so that the plan
  // replays the same schedule from its first Invoke on and the decisions can be written down at Compile.
  void Settle();
  // H2D inputs, `epoch` replays of all steps, D2H outputs; returns mean wall
  // nanoseconds per replay of the launch-and-wait loop alone (reference
  // runner.cpp:101-119). `args` maps every argument name to a host buffer of
  // exactly Meta::GetSize() bytes; a missing name throws std::out_of_range
  // (reference runner.cpp:70).
  size_t Run(const std::unordered_map<std::string, void *> &args, size_t epoch);
  // `n` replays on inputs already resident in HBM, then a stream wait; no host copies.
  void ReplayResident(size_t n);
  // kernel-exact hipEvent duration of every launch of the schedule, median of `iters` runs after `warmup`.
  std::vector<StepTime> Profile(size_t warmup, size_t iters);
  // mean device time of one whole replay measured with events on the plan's stream
  double TimeReplayNs(size_t warmup, size_t iters);
  // device time of each of `iters` consecutive replays (events between them on the plan's stream, no host waits)
  std::vector<double> ReplayTimesNs(size_t warmup, size_t iters);

  void SetFlags(uint32_t flags) { flags_ = flags; }
  uint32_t GetFlags() const { return flags_; }
  void SetUseGraph(bool use) { use_graph_ = use; }
  // launch-level fusion of single-reader chains; off whenever literal-reference flags are set
  void SetFuse(bool fuse) { fuse_ = fuse; }
  // MatMul nodes on the opt-in bf16 path (operands rounded to bf16, fp32 accumulation)
  void SetBf16(bool on) { bf16_ = on; }
  // device address of a named interface / constant operand (tests)
  void *GetDeviceAddress(const std::string &name) const;
  void *GetArenaBase() const { return arena_; }
  void *GetStream() const { return stream_; }
  // Two runs of launches that follow each other in the schedule, [a_begin, b_begin) and [b_begin, end), the second
  // of which reads nothing the first writes: the second run is issued on a stream beside the plan's, between a fork
  // in front of the first run and a join behind the second, and everything it writes lives in buffers of its own
  // instead of the memory plan's bytes (which the first run may still be using).
  struct Region {
    size_t a_begin = 0, b_begin = 0, end = 0;
  };
  const std::vector<Region> &GetRegions() const {
    GetSchedule();
    return regions_;
  }
  // a region is formed when the shorter of its two runs is estimated at least this long (microseconds)
  void SetBranchMinUs(double us) { branch_min_us_ = us; }
  // whether the first run times the schedule with and without its regions and keeps the faster one
  void SetBranchCheck(bool on) { branch_check_ = on; }
  // 1 / 0: keep / drop the side branches without timing them (a decision read back from an earlier compile's JSON);
  // negative: decide by timing
  void SetBranchDecision(int keep) { branch_decision_ = keep; }
  // 1 / 0 once the first run has decided (or a decision was given), -1 before, or when there was nothing to decide
  int GetBranchDecision() const { return branches_decided_ && had_regions_ ? (branches_off_ ? 0 : 1) : -1; }

  // The table the contraction launches take their tile configuration from; in its Measure mode, signatures it does
  // not hold yet are timed inside this plan's schedule when the plan is materialised (reference: the generators'
  // autotune, src/structure/kernel/generator/matmul.cpp:88-131).
  void SetContractionTable(std::shared_ptr<kernel::ContractionTable> table) { table_ = std::move(table); }
  // signature of schedule entry `i` in the ContractionTable; empty when the launch is no MatMul / Gemm
  std::string ContractionSignature(size_t i) const;
  // (signature, FL_CONTRACT_* bits in use) of every contraction launch of the schedule, in schedule order
  std::vector<std::pair<std::string, uint32_t>> GetContractionChoices() const;

 private:
  struct ConstantSlot {
    Tensor tensor;
    std::vector<size_t> layout;
    void *device = nullptr;
  };
  struct RawSlot {
    size_t bytes = 0;
    void *device = nullptr;
  };
  void *Resolve(const Operand &op) const;
  void IssueStep(kernel::LaunchContext &ctx, const Step &s, const Operand *in0_view = nullptr,
                 const Operand *in1_view = nullptr, const Operand *out_view = nullptr, int *rc_out = nullptr) const;
  // `rc_out` given: a refusal of the C ABI is stored there instead of being thrown (tuning probes)
  void Issue(kernel::LaunchContext &ctx, const Launch &l, int *rc_out = nullptr) const;
  void TuneContractions();
  void ApplyContractionPicks() const;
  // LayerNormalizations the schedule keeps out of memory: private buffers for their row statistics (host side) ...
  void PlanNormBuffers() const;
  // ... and, once per plan, the scale folded into the weights of the contractions that read them, with the two
  // per-column vectors their epilogue needs (new constants "norm_c1:<weights>" and "norm_c2:<weights>")
  void FoldNorms();
  void LaunchAll(kernel::LaunchContext &ctx) const;
  void Replay(kernel::LaunchContext &ctx);
  void PlanBranches() const;
  void DecideBranches();

  std::string name_;
  size_t arena_bytes_;
  std::vector<Argument> arguments_;
  std::vector<Step> steps_;
  std::map<std::string, ConstantSlot> constants_;
  mutable std::map<std::string, RawSlot> privates_;
  std::map<std::string, RawSlot> interfaces_;
  uint32_t flags_ = 0;
  bool use_graph_ = true;
  bool fuse_ = true;
  bool bf16_ = false;
  mutable std::vector<Launch> schedule_;
  mutable bool schedule_built_ = false;
  mutable std::vector<Region> regions_;
  double branch_min_us_ = 12.0;
  bool branch_check_ = true;
  bool branches_decided_ = false;
  mutable bool branches_off_ = false;
  int branch_decision_ = -1;
  bool had_regions_ = false;
  std::shared_ptr<kernel::ContractionTable> table_;
  std::map<std::string, size_t> folded_;  // weight constants that carry a LayerNormalization's scale -> that step
  void *side_stream_ = nullptr;
  std::vector<void *> region_events_;  // fork and join event of every region
  void *arena_ = nullptr;
  void *stream_ = nullptr;
  void *graph_ = nullptr;
};

}  // namespace worker
}  // namespace fluidml

#endif
