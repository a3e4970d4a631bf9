#include "worker/launcher.h"

#include <algorithm>
#include <chrono>
#include <limits>
#include <cstdlib>
#include <map>
#include <sstream>
#include <stdexcept>

#include "fluidml_hip.h"

namespace fluidml {
namespace worker {

namespace {
void Check(int rc, const char *what) {
  if (rc != 0) throw std::runtime_error(std::string(what) + ": " + fluidml_hip_error_string(rc));
}

kernel::TensorView ViewOf(void *base, const Operand &op) {
  if (!op.viewed) return kernel::TensorView(base, op.meta, op.layout);
  kernel::TensorView v(static_cast<char *>(base) + op.view_offset * static_cast<int64_t>(GetSize(op.meta.GetType())), op.meta);
  for (size_t d = 0; d < op.view_strides.size(); ++d) v.t.strides[d] = op.view_strides[d];
  return v;
}

const char *SpaceName(Operand::Space s) {
  switch (s) {
    case Operand::Space::Arena: return "arena";
    case Operand::Space::Interface: return "interface";
    case Operand::Space::Constant: return "constant";
    default: return "private";
  }
}
}  // namespace

LaunchPlan::LaunchPlan(std::string &&name, size_t arena_bytes) : name_(std::move(name)), arena_bytes_(arena_bytes) {}

LaunchPlan::~LaunchPlan() {
  if (graph_) fluidml_hip_graph_destroy(graph_);
  for (void *e : region_events_) fluidml_hip_event_destroy(e);
  if (side_stream_) fluidml_hip_stream_destroy(side_stream_);
  for (auto &kv : constants_) fluidml_hip_free(kv.second.device);
  for (auto &kv : privates_) fluidml_hip_free(kv.second.device);
  for (auto &kv : interfaces_) fluidml_hip_free(kv.second.device);
  if (arena_) fluidml_hip_arena_destroy(arena_);
  if (stream_) fluidml_hip_stream_destroy(stream_);
}

void LaunchPlan::AddArgument(Argument &&arg) {
  interfaces_[arg.name].bytes = arg.meta.GetSize();
  arguments_.push_back(std::move(arg));
}

void LaunchPlan::AddConstant(const std::string &name, const Tensor &tensor, const std::vector<size_t> &layout) {
  constants_.insert({name, ConstantSlot{tensor, layout, nullptr}});
}

void LaunchPlan::AddPrivate(const std::string &name, size_t bytes) { privates_[name].bytes = bytes; }

void LaunchPlan::AddStep(Step &&step) { steps_.push_back(std::move(step)); }

size_t LaunchPlan::GetConstantBytes() const {
  size_t n = 0;
  for (const auto &kv : constants_) n += kv.second.tensor.GetMeta().GetSize();
  for (const Step &s : steps_) n += s.kernel->GetConstantBytes();
  return n;
}

size_t LaunchPlan::GetPrivateBytes() const {
  GetSchedule();
  size_t n = 0;
  for (const auto &kv : privates_) n += kv.second.bytes;
  return n;
}

size_t LaunchPlan::GetInterfaceBytes() const {
  size_t n = 0;
  for (const auto &kv : interfaces_) n += kv.second.bytes;
  return n;
}

void LaunchPlan::Validate() const {
  auto check_operand = [&](const Step &s, const Operand &op) {
    switch (op.space) {
      case Operand::Space::Arena:
        if (op.offset + op.meta.GetSize() > arena_bytes_) throw std::logic_error("plan: " + s.node->GetName() + " operand " + op.name + " leaves the arena");
        break;
      case Operand::Space::Interface:
        if (!interfaces_.count(op.name)) throw std::logic_error("plan: unknown interface tensor " + op.name);
        break;
      case Operand::Space::Constant:
        if (!constants_.count(op.name)) throw std::logic_error("plan: unknown constant " + op.name);
        break;
      case Operand::Space::Private:
        if (!privates_.count(op.name)) throw std::logic_error("plan: unknown private tensor " + op.name);
        break;
    }
  };
  for (const Step &s : steps_) {
    if (!s.kernel) throw std::logic_error("plan: " + s.node->GetName() + " has no kernel");
    check_operand(s, s.in0);
    if (s.node->IsDoubleInputs()) check_operand(s, s.in1);
    check_operand(s, s.out);
    if (s.has_buffer && s.buffer_offset + s.buffer_bytes > arena_bytes_) {
      throw std::logic_error("plan: scratch of " + s.node->GetName() + " leaves the arena");
    }
  }
}

std::string LaunchPlan::ToText() const {
  std::ostringstream os;
  auto operand = [&](const Operand &op) {
    os << op.name << "@" << SpaceName(op.space);
    if (op.space == Operand::Space::Arena) os << "+" << op.offset;
    os << ":" << GetStringFromType(op.meta.GetType()) << "[";
    for (size_t i = 0; i < op.meta.GetShape().size(); ++i) os << (i ? "," : "") << op.meta.GetShape()[i];
    os << "]/(";
    for (size_t i = 0; i < op.layout.size(); ++i) os << (i ? "," : "") << op.layout[i];
    os << ")";
  };
  os << "launch_plan @" << name_ << " arena_bytes=" << arena_bytes_ << " constant_bytes=" << GetConstantBytes()
     << " interface_bytes=" << GetInterfaceBytes() << "\n";
  for (const Argument &a : arguments_) {
    os << "  arg " << (a.type == Argument::Type::Input ? "in  " : "out ") << a.name << " bytes=" << a.meta.GetSize() << "\n";
  }
  for (size_t i = 0; i < steps_.size(); ++i) {
    const Step &s = steps_[i];
    os << "  %" << i << " " << s.kernel->GetKernelName() << " \"" << s.node->GetName() << "\" (";
    operand(s.in0);
    if (s.node->IsDoubleInputs()) {
      os << ", ";
      operand(s.in1);
    }
    os << ") -> ";
    operand(s.out);
    if (s.has_buffer) os << " scratch@arena+" << s.buffer_offset << ":" << s.buffer_bytes;
    os << "\n";
  }
  const std::vector<Launch> &schedule = GetSchedule();
  size_t run = 0;
  for (const Launch &l : schedule) run += l.kind != Launch::Kind::View && l.kind != Launch::Kind::Placed ? 1 : 0;
  os << "  schedule launches=" << run << "\n";
  for (const Launch &l : schedule) {
    if (l.kind == Launch::Kind::Step) continue;
    os << "    fused " << LaunchKindName(l.kind) << " {";
    for (size_t m = 0; m < l.members.size(); ++m) os << (m ? "," : "") << "%" << l.members[m];
    os << "}\n";
  }
  return os.str();
}

void LaunchPlan::Materialize() {
  if (arena_ != nullptr) return;
  Validate();
  GetSchedule();  // may move tensors of a side branch into buffers of their own, allocated below
  FoldNorms();
  Check(fluidml_hip_stream_create(&stream_), "creating the plan's stream");
  if (!regions_.empty()) {
    Check(fluidml_hip_stream_create(&side_stream_), "creating the plan's second stream");
    region_events_.resize(2 * regions_.size(), nullptr);
    for (void *&e : region_events_) Check(fluidml_hip_event_create(&e), "creating a fork/join event");
  }
  for (auto &kv : constants_) {
    const std::vector<uint8_t> bytes = kv.second.tensor.Pack(kv.second.layout, (flags_ & FL_REF_CONSTANT_GATHERED) != 0);
    Check(fluidml_hip_upload_constant(bytes.data(), bytes.size(), &kv.second.device), "uploading a constant region");
  }
  for (auto *slots : {&privates_, &interfaces_}) {
    for (auto &kv : *slots) Check(fluidml_hip_arena_create(kv.second.bytes, &kv.second.device), "allocating a device buffer");
  }
  for (Step &s : steps_) s.kernel->Prepare();
  Check(fluidml_hip_arena_create(arena_bytes_, &arena_), "allocating the arena");
  TuneContractions();
}

void *LaunchPlan::Resolve(const Operand &op) const {
  switch (op.space) {
    case Operand::Space::Arena: return static_cast<char *>(arena_) + op.offset;
    case Operand::Space::Interface: return interfaces_.at(op.name).device;
    case Operand::Space::Constant: return constants_.at(op.name).device;
    default: {
      const auto it = privates_.find(op.pool.empty() ? op.name : op.pool);
      if (it == privates_.end()) throw std::logic_error("plan: no buffer outside the arena for " + op.name);
      return static_cast<char *>(it->second.device) + op.offset;
    }
  }
}

void *LaunchPlan::GetDeviceAddress(const std::string &name) const {
  auto it = interfaces_.find(name);
  if (it != interfaces_.end()) return it->second.device;
  auto ct = constants_.find(name);
  if (ct != constants_.end()) return ct->second.device;
  return nullptr;
}

const std::vector<Launch> &LaunchPlan::GetSchedule() const {
  if (!schedule_built_) {
    schedule_ = BuildSchedule(steps_, fuse_ && flags_ == 0);
    schedule_built_ = true;
    regions_.clear();
    if (fuse_ && flags_ == 0 && !branches_off_) PlanBranches();
    PlanNormBuffers();
  }
  return schedule_;
}

void LaunchPlan::PlanNormBuffers() const {
  // tensors the schedule moved out of the arena (the plan's bytes for them are in use when the fused launch writes
  // or reads them): a buffer each, named like the tensor
  auto moved_out = [&](const Operand &out) {
    // (a launch that writes a part of the tensor -- an input of a Concat2 placed in its output -- names the whole)
    if (out.space != Operand::Space::Private || !out.pool.empty() || out.name.empty()) return;
    size_t &bytes = privates_[out.name].bytes;
    bytes = std::max(bytes, out.viewed ? out.source_bytes : out.meta.GetSize());
  };
  for (const Launch &l : schedule_) {
    if (l.kind != Launch::Kind::View && l.kind != Launch::Kind::Placed && (l.kind != Launch::Kind::Step || l.rewired)) {
      if (l.group.empty()) moved_out(l.out);
      if (l.has_out2) moved_out(l.out2);
      for (const Launch &m : l.group) moved_out(m.out);
    }
    if (l.norm_stats_out.empty()) continue;
    const std::vector<int64_t> &shape = l.out.meta.GetShape();
    size_t rows = 1;
    for (size_t d = 0; d + 1 < shape.size(); ++d) rows *= static_cast<size_t>(shape[d]);
    const size_t parts = (static_cast<size_t>(shape.back()) + 31) / 32;
    privates_[l.norm_stats_out].bytes = rows * parts * 2 * sizeof(float);  // (mean, M2) per run of 32 columns
  }
}

void LaunchPlan::FoldNorms() {
  auto fold = [&](const Launch &m, size_t owner) {
    const std::string &wname = m.b.name;
    auto done = folded_.find(wname);
    if (done != folded_.end()) {
      if (done->second != owner) throw std::logic_error("plan: weights " + wname + " serve two LayerNormalizations");
      return;
    }
    ConstantSlot &w = constants_.at(wname);
    const flow::Attrs &at = steps_[owner].node->GetAttrs();
    if (!at.t0 || !at.t1) throw std::logic_error("plan: the deferred LayerNormalization holds no scale / shift");
    const std::vector<float64_t> &scale = at.t0->Get(), &shift = at.t1->Get(), &old = w.tensor.Get();
    const std::vector<int64_t> &shape = w.tensor.GetShape();
    const size_t K = static_cast<size_t>(shape[0]), N = static_cast<size_t>(shape[1]);
    if (scale.size() != K || shift.size() != K) throw std::logic_error("plan: LayerNormalization width and weight rows differ");
    std::vector<float64_t> scaled(old.size()), c1(N, 0.0), c2(N, 0.0);
    for (size_t k = 0; k < K; ++k) {
      for (size_t n = 0; n < N; ++n) {
        // the product is what the device multiplies with, so the column sums use its fp32 value
        const float64_t v = static_cast<float64_t>(static_cast<float>(scale[k] * old[k * N + n]));
        scaled[k * N + n] = v;
        c1[n] += v;
        c2[n] += shift[k] * old[k * N + n];
      }
    }
    if (m.has_c) {
      const std::vector<float64_t> &bias = constants_.at(m.c.name).tensor.Get();
      for (size_t n = 0; n < N; ++n) c2[n] += bias[n];
    }
    w.tensor = Tensor(Type::kFloat32, std::vector<int64_t>(shape), std::move(scaled));
    constants_.insert({"norm_c1:" + wname, ConstantSlot{Tensor(Type::kFloat32, {static_cast<int64_t>(N)}, std::move(c1)), {0}, nullptr}});
    constants_.insert({"norm_c2:" + wname, ConstantSlot{Tensor(Type::kFloat32, {static_cast<int64_t>(N)}, std::move(c2)), {0}, nullptr}});
    folded_[wname] = owner;
  };
  for (const Launch &l : GetSchedule()) {
    if (l.norm_mode != 1) continue;
    if (l.kind == Launch::Kind::MatMulGroup) {
      for (const Launch &m : l.group) fold(m, l.norm_owner);
    } else {
      fold(l, l.norm_owner);
    }
  }
}

namespace {
bool Alias(const Operand &x, const Operand &y) {
  if (x.space != y.space) return false;
  if (x.space == Operand::Space::Interface || x.space == Operand::Space::Constant) return x.name == y.name;
  if (x.space == Operand::Space::Private && (x.pool.empty() ? x.name : x.pool) != (y.pool.empty() ? y.name : y.pool)) return false;
  return x.offset < y.offset + y.Extent() && y.offset < x.offset + x.Extent();  // bytes of the arena / of one buffer
}

// the operands a launch reads and writes (pointers into the launch, so that they can be redirected)
struct Access {
  std::vector<Operand *> reads, writes;
  bool runs = true;     // false: a view or a step whose bytes are already in place
  double cost_us = 0;
};

bool BranchesEnabled() {
  const char *v = std::getenv("FLUIDML_BRANCHES");  // (read at every compile)
  return v == nullptr || std::strtol(v, nullptr, 10) != 0;
}
}  // namespace

// Looks for pairs of consecutive runs of launches A, B where B reads nothing A writes (attention block and MLP of a
// parallel-residual layer, convolution branch and attention branch of a mixed-attention layer) and lets B run on a
// second stream beside A.  The memory plan was made for the serial order, so bytes B writes may be ones A still
// uses: every tensor B writes moves to a buffer of its own, and its readers with it.
// (The scratch the memory plan reserves for some steps is not touched by any kernel here unless literal-reference
// flags are set, and then no branches are planned.)
void LaunchPlan::PlanBranches() const {
  regions_.clear();
  if (!BranchesEnabled()) return;
  std::vector<Launch> &sched = schedule_;
  const size_t n = sched.size();
  // every single step carries its operands itself from here on, so that they can be redirected
  for (Launch &l : sched) {
    if (l.kind == Launch::Kind::Step && !l.rewired) {
      const Step &st = steps_[l.members[0]];
      l.rewired = true;
      l.a = st.in0;
      if (st.node->IsDoubleInputs()) l.b = st.in1;
      l.out = st.out;
    }
  }
  std::vector<Access> acc(n);
  auto add_reads = [](Access &a, Launch &l) {
    for (Operand *op : {&l.a, &l.b, &l.c, &l.d, &l.e}) {
      if (!op->name.empty() && op->space != Operand::Space::Constant) a.reads.push_back(op);
    }
  };
  for (size_t i = 0; i < n; ++i) {
    Launch &l = sched[i];
    Access &a = acc[i];
    if (l.kind == Launch::Kind::View || l.kind == Launch::Kind::Placed) {
      a.runs = false;
      continue;
    }
    add_reads(a, l);
    if (l.group.empty()) {
      a.writes.push_back(&l.out);
    } else {
      for (Launch &g : l.group) {
        add_reads(a, g);
        a.writes.push_back(&g.out);
      }
    }
    if (l.has_out2) a.writes.push_back(&l.out2);
    // a launch is a few microseconds of latency plus its work at a fraction of the peaks
    a.cost_us = 4.0 + l.flops / 6e7 + l.bytes / 3e6;
  }
  // writers of every arena tensor
  std::map<std::string, std::vector<size_t>> writers;
  for (size_t i = 0; i < n; ++i) {
    for (const Operand *w : acc[i].writes) {
      if (w->space == Operand::Space::Arena) writers[w->name].push_back(i);
    }
  }
  // A fork and a join cost about 18 us on this runtime (measured on captured graphs: a region whose runs take 10 us
  // each replays 6 us slower than the same launches in a row, one with 40 us runs 22 us faster), so only runs of some
  // length are candidates; whether the candidates stay is decided by timing the schedule (DecideBranches).
  constexpr size_t kMaxRun = 10;
  const char *min_us_switch = std::getenv("FLUIDML_BRANCH_MIN_US");
  const double env_min_us = min_us_switch != nullptr ? std::strtod(min_us_switch, nullptr) : -1.0;
  const double min_us = env_min_us >= 0 ? env_min_us : branch_min_us_;
  auto eligible = [&](size_t a0, size_t b0, size_t e) {
    for (size_t y = b0; y < e; ++y) {
      if (!acc[y].runs) continue;
      for (const Operand *r : acc[y].reads) {
        // what B produces itself moves out of the arena with its writers (checked below): no bytes shared with A
        if (r->space == Operand::Space::Arena) {
          auto it = writers.find(r->name);
          if (it != writers.end() && !it->second.empty() && it->second.front() >= b0 && it->second.back() < e) continue;
        }
        for (size_t x = a0; x < b0; ++x) {
          for (const Operand *w : acc[x].writes) {
            if (Alias(*w, *r)) return false;
          }
        }
      }
      for (const Operand *w : acc[y].writes) {
        if (w->space == Operand::Space::Arena) {
          for (size_t wr : writers[w->name]) {
            if (wr < b0 || wr >= e) return false;  // written elsewhere too: has to stay in the plan's bytes
          }
        } else {
          // a graph output, or a buffer of its own already: nothing of A may touch it
          for (size_t x = a0; x < b0; ++x) {
            for (const Operand *o : acc[x].reads) {
              if (Alias(*w, *o)) return false;
            }
            for (const Operand *o : acc[x].writes) {
              if (Alias(*w, *o)) return false;
            }
          }
        }
      }
    }
    return true;
  };
  std::vector<size_t> side_free_from;  // per shared buffer: first launch index from which nobody uses its contents
  size_t i = 0;
  while (i < n) {
    if (!acc[i].runs) {
      ++i;
      continue;
    }
    double best_gain = std::max(0.0, min_us) - 1e-9;  // the shorter run's estimate has to reach this
    size_t best_b = 0, best_e = 0;
    double cost_a = 0;
    size_t runs_a = 0;
    for (size_t b0 = i + 1; b0 < n && runs_a < kMaxRun; ++b0) {
      if (acc[b0 - 1].runs) {
        cost_a += acc[b0 - 1].cost_us;
        ++runs_a;
      }
      if (!acc[b0].runs) continue;  // B starts at a launch that runs
      double cost_b = 0;
      size_t runs_b = 0;
      for (size_t e = b0 + 1; e <= n && runs_b < kMaxRun; ++e) {
        if (!acc[e - 1].runs) continue;
        cost_b += acc[e - 1].cost_us;
        ++runs_b;
        const double gain = std::min(cost_a, cost_b);
        if (gain <= best_gain) continue;
        if (!eligible(i, b0, e)) continue;  // (a longer B may take in the other writer of a tensor)
        best_gain = gain;
        best_b = b0;
        best_e = e;
      }
    }
    if (best_e == 0) {
      ++i;
      continue;
    }
    regions_.push_back({i, best_b, best_e});
    // Move what B writes out of the arena, into a buffer the side branches share: a region takes the first of the
    // buffers whose previous tenants nobody touches from this region's fork on (B starts right behind the fork).
    struct Moved {
      size_t bytes = 0, offset = 0, last_use = 0;
    };
    std::map<std::string, Moved> moved;
    for (size_t y = best_b; y < best_e; ++y) {
      for (const Operand *w : acc[y].writes) {
        if (w->space == Operand::Space::Arena) moved[w->name].bytes = std::max(moved[w->name].bytes, w->Extent());
      }
    }
    size_t last_use = best_e;
    for (size_t k = 0; k < n; ++k) {
      Launch &l = sched[k];
      auto touch = [&](Launch &x) {
        for (Operand *op : {&x.a, &x.b, &x.c, &x.d, &x.e, &x.out, &x.out2}) {
          if (op->space != Operand::Space::Arena || op->name.empty()) continue;
          auto it = moved.find(op->name);
          if (it == moved.end()) continue;
          it->second.bytes = std::max(it->second.bytes, op->Extent());
          last_use = std::max(last_use, k);
        }
      };
      touch(l);
      for (Launch &g : l.group) touch(g);
    }
    size_t total = 0;
    for (auto &kv : moved) {
      kv.second.offset = total;
      total += (kv.second.bytes + 255) / 256 * 256;
    }
    size_t slot = 0;
    while (slot < side_free_from.size() && side_free_from[slot] > i) ++slot;
    if (slot == side_free_from.size()) side_free_from.push_back(0);
    side_free_from[slot] = last_use + 1;
    const std::string buffer = "side:" + std::to_string(slot);
    privates_[buffer].bytes = std::max(privates_[buffer].bytes, total);
    for (Launch &l : sched) {
      auto redirect = [&](Launch &x) {
        for (Operand *op : {&x.a, &x.b, &x.c, &x.d, &x.e, &x.out, &x.out2}) {
          if (op->space != Operand::Space::Arena || op->name.empty()) continue;
          auto it = moved.find(op->name);
          if (it == moved.end()) continue;
          op->space = Operand::Space::Private;
          op->pool = buffer;
          op->offset = it->second.offset;
        }
      };
      redirect(l);
      for (Launch &g : l.group) redirect(g);
    }
    i = best_e;
  }
}

void LaunchPlan::IssueStep(kernel::LaunchContext &ctx, const Step &s, const Operand *in0_view,
                           const Operand *in1_view, const Operand *out_view, int *rc_out) const {
  const Operand &op0 = in0_view ? *in0_view : s.in0, &opo = out_view ? *out_view : s.out;
  const kernel::TensorView in0 = ViewOf(Resolve(op0), op0), out = ViewOf(Resolve(opo), opo);
  const kernel::Buffer buffer{s.has_buffer ? static_cast<char *>(arena_) + s.buffer_offset : nullptr, s.buffer_bytes};
  kernel::Kernel *k = s.kernel.get();
  if (s.node->IsSingleInput()) {
    if (s.has_buffer) dynamic_cast<kernel::SingleInputWithBufferKernel &>(*k).Run(ctx, in0, out, buffer);
    else dynamic_cast<kernel::SingleInputWithoutBufferKernel &>(*k).Run(ctx, in0, out);
  } else {
    const Operand &op1 = in1_view ? *in1_view : s.in1;
    const kernel::TensorView in1 = ViewOf(Resolve(op1), op1);
    if (s.has_buffer) dynamic_cast<kernel::DoubleInputsWithBufferKernel &>(*k).Run(ctx, in0, in1, out, buffer);
    else dynamic_cast<kernel::DoubleInputsWithoutBufferKernel &>(*k).Run(ctx, in0, in1, out);
  }
  if (rc_out != nullptr) {
    *rc_out = ctx.status;
    ctx.status = 0;
    ctx.failed.clear();
    return;
  }
  if (ctx.status != 0) {
    throw std::runtime_error("launching " + ctx.failed + " for node '" + s.node->GetName() + "': " +
                             fluidml_hip_error_string(ctx.status));
  }
}

namespace {
// `t` seen through a transpose: result[k] walks t's dim perm[k]
fl_tensor Permuted(const fl_tensor &t, const std::vector<int64_t> &perm, bool inverse) {
  fl_tensor v = t;
  for (int32_t k = 0; k < t.rank; ++k) {
    const int64_t p = perm.empty() ? t.rank - 1 - k : perm[static_cast<size_t>(k)];
    if (inverse) {
      v.shape[p] = t.shape[k];
      v.strides[p] = t.strides[k];
    } else {
      v.shape[k] = t.shape[p];
      v.strides[k] = t.strides[p];
    }
  }
  return v;
}
}  // namespace

void LaunchPlan::Issue(kernel::LaunchContext &ctx, const Launch &l, int *rc_out) const {
  if (rc_out != nullptr) *rc_out = 0;
  if (l.kind == Launch::Kind::View || l.kind == Launch::Kind::Placed) return;  // nothing runs
  if (l.kind == Launch::Kind::Step) {
    const uint32_t before = ctx.contract;
    ctx.contract = l.contract;
    IssueStep(ctx, steps_[l.members[0]], l.rewired ? &l.a : nullptr, l.rewired ? &l.b : nullptr,
              l.rewired ? &l.out : nullptr, rc_out);
    ctx.contract = before;
    return;
  }
  const kernel::TensorView a = ViewOf(Resolve(l.a), l.a), out = ViewOf(Resolve(l.out), l.out);
  const uint32_t contract_flags = (ctx.bf16 ? FL_CONTRACT_BF16 : 0u) | l.contract;
  int rc = FL_ERR_UNSUPPORTED;
  switch (l.kind) {
    case Launch::Kind::MatMulChain: {
      const kernel::TensorView b = ViewOf(Resolve(l.b), l.b);
      kernel::TensorView c;
      if (l.has_c) c = ViewOf(Resolve(l.c), l.c);
      if (l.norm_mode != 0 || !l.norm_stats_out.empty()) {
        // a LayerNormalization folded into the launch: see DeferLayerNorms in fusion.cpp
        kernel::TensorView d, e, c1, c2, dst = out;
        if (l.has_skip) d = ViewOf(Resolve(l.d), l.d);
        if (l.has_skip2) e = ViewOf(Resolve(l.e), l.e);
        if (!l.view_strides.empty()) {
          dst = kernel::TensorView(out.t.base, steps_[l.members[0]].out.meta);
          for (size_t k = 0; k < l.view_strides.size(); ++k) dst.t.strides[k] = l.view_strides[k];
        }
        fl_norm_fusion norm{};
        kernel::TensorView scale, shift;
        const fl_tensor *bias = l.has_c ? &c.t : nullptr, *col_sum = nullptr;
        if (l.norm_mode != 0) {
          const Step &owner = steps_[l.norm_owner];
          norm.deferred = l.norm_mode;
          norm.epsilon = owner.node->GetAttrs().epsilon;
          norm.stats = static_cast<const float *>(privates_.at(l.norm_stats).device);
          if (l.norm_mode == FL_NORM_LHS) {
            norm.width = static_cast<int32_t>(l.a.meta.GetShape().back());
            const ConstantSlot &s1 = constants_.at("norm_c1:" + l.b.name), &s2 = constants_.at("norm_c2:" + l.b.name);
            c1 = kernel::TensorView(s1.device, s1.tensor.GetMeta());
            c2 = kernel::TensorView(s2.device, s2.tensor.GetMeta());
            col_sum = &c1.t;
            bias = &c2.t;
          } else {
            norm.width = static_cast<int32_t>(l.d.meta.GetShape().back());
            scale = owner.kernel->GetConstant(0)->View();
            shift = owner.kernel->GetConstant(1)->View();
            norm.scale = &scale.t;
            norm.shift = &shift.t;
          }
        }
        if (!l.norm_stats_out.empty()) norm.stats_out = static_cast<float *>(privates_.at(l.norm_stats_out).device);
        if (l.has_skip2) norm.addend2 = &e.t;
        const fl_tensor *rhs_p = &b.t, *dst_p = &dst.t;
        rc = fluidml_hip_matmul_chain_group_norm(1, &a.t, &rhs_p, &bias, col_sum != nullptr ? &col_sum : nullptr, &dst_p, l.n_inner,
                                                 &l.stride_outer, &l.chain, l.has_skip ? &d.t : nullptr, &norm, contract_flags,
                                                 ctx.stream);
        break;
      }
      if (l.has_skip) {
        const kernel::TensorView d = ViewOf(Resolve(l.d), l.d);
        kernel::TensorView e;
        if (l.has_skip2) e = ViewOf(Resolve(l.e), l.e);
        rc = fluidml_hip_matmul_chain_add(&a.t, &b.t, l.has_c ? &c.t : nullptr, &out.t, &l.chain, &d.t,
                                          l.has_skip2 ? &e.t : nullptr, contract_flags, ctx.stream);
      } else if (l.view_strides.empty()) {
        rc = fluidml_hip_matmul_chain(&a.t, &b.t, l.has_c ? &c.t : nullptr, &out.t, &l.chain, contract_flags, ctx.stream);
      } else {
        // the contraction's logical output addressed inside the buffer of the last folded Reshape / Transpose
        kernel::TensorView dst(out.t.base, steps_[l.members[0]].out.meta);
        for (size_t d = 0; d < l.view_strides.size(); ++d) dst.t.strides[d] = l.view_strides[d];
        rc = fluidml_hip_matmul_chain_view(&a.t, &b.t, l.has_c ? &c.t : nullptr, &dst.t, l.n_inner, l.stride_outer,
                                           &l.chain, contract_flags, ctx.stream);
      }
      break;
    }
    case Launch::Kind::MatMulGroup: {
      const size_t n = l.group.size();
      std::vector<kernel::TensorView> rhs(n), bias(n), dst(n);
      std::vector<const fl_tensor *> rhs_p(n), bias_p(n), dst_p(n);
      std::vector<int64_t> outer(n);
      for (size_t g = 0; g < n; ++g) {
        const Launch &m = l.group[g];
        rhs[g] = ViewOf(Resolve(m.b), m.b);
        if (m.has_c) bias[g] = ViewOf(Resolve(m.c), m.c);
        if (m.view_strides.empty()) {
          dst[g] = ViewOf(Resolve(m.out), m.out);
        } else {
          dst[g] = kernel::TensorView(Resolve(m.out), steps_[m.members[0]].out.meta);
          for (size_t d = 0; d < m.view_strides.size(); ++d) dst[g].t.strides[d] = m.view_strides[d];
        }
        rhs_p[g] = &rhs[g].t;
        bias_p[g] = m.has_c ? &bias[g].t : nullptr;
        dst_p[g] = &dst[g].t;
        outer[g] = m.stride_outer;
      }
      if (l.norm_mode == FL_NORM_LHS) {
        // the shared left operand is the un-normalised input of a LayerNormalization that is not run
        std::vector<kernel::TensorView> c1(n), c2(n);
        std::vector<const fl_tensor *> c1_p(n), c2_p(n);
        for (size_t g = 0; g < n; ++g) {
          const ConstantSlot &s1 = constants_.at("norm_c1:" + l.group[g].b.name), &s2 = constants_.at("norm_c2:" + l.group[g].b.name);
          c1[g] = kernel::TensorView(s1.device, s1.tensor.GetMeta());
          c2[g] = kernel::TensorView(s2.device, s2.tensor.GetMeta());
          c1_p[g] = &c1[g].t;
          c2_p[g] = &c2[g].t;
        }
        fl_norm_fusion norm{};
        norm.deferred = FL_NORM_LHS;
        norm.width = static_cast<int32_t>(l.a.meta.GetShape().back());
        norm.epsilon = steps_[l.norm_owner].node->GetAttrs().epsilon;
        norm.stats = static_cast<const float *>(privates_.at(l.norm_stats).device);
        rc = fluidml_hip_matmul_chain_group_norm(static_cast<int32_t>(n), &a.t, rhs_p.data(), c2_p.data(), c1_p.data(), dst_p.data(),
                                                 l.group[0].n_inner, outer.data(), &l.group[0].chain, nullptr, &norm,
                                                 contract_flags, ctx.stream);
        break;
      }
      rc = fluidml_hip_matmul_chain_group(static_cast<int32_t>(n), &a.t, rhs_p.data(), bias_p.data(), dst_p.data(),
                                          l.group[0].n_inner, outer.data(), &l.group[0].chain, contract_flags,
                                          ctx.stream);
      break;
    }
    case Launch::Kind::GemmChain: {
      const kernel::TensorView b = ViewOf(Resolve(l.b), l.b);
      const flow::Attrs &at = steps_[l.owner].node->GetAttrs();
      const kernel::DeviceConstant *bias = steps_[l.owner].kernel->GetConstant(0);
      if (bias == nullptr) throw std::logic_error("fused Gemm: the node holds no bias");
      const kernel::TensorView c = bias->View();
      rc = fluidml_hip_gemm_chain(&a.t, &b.t, &c.t, &out.t, at.alpha, at.beta, at.trans_a ? 1 : 0, at.trans_b ? 1 : 0,
                                  &l.chain, contract_flags, ctx.stream);
      break;
    }
    case Launch::Kind::ConvChain: {
      const kernel::TensorView b = ViewOf(Resolve(l.b), l.b);
      const flow::Attrs &at = steps_[l.owner].node->GetAttrs();
      const kernel::DeviceConstant *bias = steps_[l.owner].kernel->GetConstant(0);
      kernel::TensorView c;
      if (bias != nullptr) c = bias->View();
      const bool padded = steps_[l.owner].node->GetKind() == flow::OpKind::ConvWithPadding;
      if (l.has_out2) {
        const kernel::TensorView mean = ViewOf(Resolve(l.out2), l.out2);
        rc = fluidml_hip_conv_chain_mean(&a.t, &b.t, bias ? &c.t : nullptr, &out.t, padded ? at.pads.data() : nullptr,
                                         at.strides.data(), at.dilations.data(), at.group, &l.chain, &mean.t, contract_flags,
                                         ctx.stream);
        break;
      }
      if (l.has_gate || l.has_skip) {
        kernel::TensorView gate, skip;
        if (l.has_gate) gate = ViewOf(Resolve(l.c), l.c);
        if (l.has_skip) skip = ViewOf(Resolve(l.d), l.d);
        rc = fluidml_hip_conv_chain_scale_add(&a.t, &b.t, bias ? &c.t : nullptr, &out.t, padded ? at.pads.data() : nullptr,
                                              at.strides.data(), at.dilations.data(), at.group, &l.chain,
                                              l.has_gate ? &gate.t : nullptr, l.has_skip ? &skip.t : nullptr,
                                              contract_flags | (l.skip_is_factor ? FL_CONTRACT_ADDEND_IS_FACTOR : 0u), ctx.stream);
        break;
      }
      rc = fluidml_hip_conv_chain(&a.t, &b.t, bias ? &c.t : nullptr, &out.t, padded ? at.pads.data() : nullptr,
                                  at.strides.data(), at.dilations.data(), at.group, &l.chain, contract_flags, ctx.stream);
      break;
    }
    case Launch::Kind::SoftmaxMatVec: {
      const kernel::TensorView b = ViewOf(Resolve(l.b), l.b);
      if (l.view_strides.empty()) {
        rc = fluidml_hip_softmax_matvec(&a.t, &b.t, &out.t, ctx.stream);
      } else {
        kernel::TensorView dst(out.t.base, steps_[l.owner].out.meta);
        for (size_t d = 0; d < l.view_strides.size(); ++d) dst.t.strides[d] = l.view_strides[d];
        if (l.n_inner != 0) {
          // the batch dim in two parts (written into a part of a Concat2's output): [outer, inner, rows, 1]
          const int64_t batch = dst.t.shape[0];
          dst.t.rank = 4;
          dst.t.shape[3] = dst.t.shape[2];
          dst.t.strides[3] = dst.t.strides[2];
          dst.t.shape[2] = dst.t.shape[1];
          dst.t.strides[2] = dst.t.strides[1];
          dst.t.shape[1] = l.n_inner;
          dst.t.strides[1] = dst.t.strides[0];
          dst.t.shape[0] = batch / l.n_inner;
          dst.t.strides[0] = l.stride_outer;
        }
        rc = fluidml_hip_softmax_matvec(&a.t, &b.t, &dst.t, ctx.stream);
      }
      break;
    }
    case Launch::Kind::ConvPair: {
      const kernel::TensorView w1 = ViewOf(Resolve(l.b), l.b), w2 = ViewOf(Resolve(l.c), l.c);
      const kernel::DeviceConstant *bias1 = steps_[l.owner].kernel->GetConstant(0);
      const kernel::DeviceConstant *bias2 = steps_[l.owner2].kernel->GetConstant(0);
      kernel::TensorView b1, b2;
      if (bias1 != nullptr) b1 = bias1->View();
      if (bias2 != nullptr) b2 = bias2->View();
      rc = fluidml_hip_pointwise_conv_pair(&a.t, &w1.t, bias1 ? &b1.t : nullptr, &l.chain, &w2.t, bias2 ? &b2.t : nullptr,
                                           &l.chain2, &out.t, ctx.stream);
      break;
    }
    case Launch::Kind::ElementwiseChain:
      rc = fluidml_hip_elementwise_chain(&a.t, &out.t, &l.chain, ctx.stream);
      break;
    case Launch::Kind::MulAdd: {
      const kernel::TensorView b = ViewOf(Resolve(l.b), l.b), c = ViewOf(Resolve(l.c), l.c);
      rc = fluidml_hip_mul_add(&a.t, &b.t, &c.t, &out.t, ctx.stream);
      break;
    }
    case Launch::Kind::GatherAdd: {
      const kernel::DeviceConstant *table = steps_[l.owner].kernel->GetConstant(0);
      if (table == nullptr) throw std::logic_error("fused Gather: the node holds no data tensor");
      const kernel::TensorView data = table->View(), b = ViewOf(Resolve(l.b), l.b);
      if (l.has_c) {
        const kernel::TensorView c = ViewOf(Resolve(l.c), l.c);
        rc = fluidml_hip_gather_constant_data_tensor_add_tensor_lhs_add_tensor_lhs(&a.t, &data.t, &b.t, &c.t, &out.t, ctx.stream);
      } else {
        rc = fluidml_hip_gather_constant_data_tensor_add(&a.t, &data.t, &b.t, &out.t, ctx.stream);
      }
      break;
    }
    case Launch::Kind::AddAdd: {
      const kernel::TensorView b = ViewOf(Resolve(l.b), l.b), c = ViewOf(Resolve(l.c), l.c);
      rc = fluidml_hip_add_add(&a.t, &b.t, &c.t, &out.t, ctx.stream);
      break;
    }
    case Launch::Kind::Rotary: {
      const kernel::TensorView b = ViewOf(Resolve(l.b), l.b), c = ViewOf(Resolve(l.c), l.c);
      // a folded Transpose: its output buffer addressed by the untransposed logical index
      const fl_tensor dst = l.perm.empty() ? out.t : Permuted(out.t, l.perm, true);
      rc = fluidml_hip_rotary(&a.t, &b.t, &c.t, &dst, l.axis, ctx.stream);
      break;
    }
    case Launch::Kind::RotaryPair: {
      const kernel::TensorView b = ViewOf(Resolve(l.b), l.b), c = ViewOf(Resolve(l.c), l.c);
      const Launch &m0 = l.group[0], &m1 = l.group[1];
      const kernel::TensorView x0 = ViewOf(Resolve(m0.a), m0.a), o0 = ViewOf(Resolve(m0.out), m0.out);
      const kernel::TensorView x1 = ViewOf(Resolve(m1.a), m1.a), o1 = ViewOf(Resolve(m1.out), m1.out);
      const fl_tensor d0 = m0.perm.empty() ? o0.t : Permuted(o0.t, m0.perm, true);
      const fl_tensor d1 = m1.perm.empty() ? o1.t : Permuted(o1.t, m1.perm, true);
      rc = fluidml_hip_rotary_pair(&x0.t, &d0, &x1.t, &d1, &b.t, &c.t, l.axis, ctx.stream);
      break;
    }
    case Launch::Kind::DivAddSoftmax: {
      const kernel::TensorView b = ViewOf(Resolve(l.b), l.b);
      rc = fluidml_hip_div_add_softmax(&a.t, l.s0, &b.t, &out.t, l.axis, ctx.stream);
      break;
    }
    case Launch::Kind::Attention: {
      const kernel::TensorView kt = ViewOf(Resolve(l.b), l.b), v = ViewOf(Resolve(l.c), l.c);
      kernel::TensorView mask, cond;
      if (l.has_mask) mask = ViewOf(Resolve(l.d), l.d);
      if (l.has_cond) {
        const kernel::DeviceConstant *c = steps_[l.owner].kernel->GetConstant(0);
        if (c == nullptr) throw std::logic_error("fused attention: the Where node holds no condition");
        cond = c->View();
      }
      kernel::TensorView dst = out;
      if (!l.view_strides.empty()) {
        // the context's logical dims addressed inside the buffer of the last folded Transpose / Reshape
        size_t pv = 0;
        for (size_t m : l.members) {
          if (steps_[m].node->GetKind() == flow::OpKind::MatMul) pv = m;
        }
        dst = kernel::TensorView(out.t.base, steps_[pv].out.meta);
        for (size_t d = 0; d < l.view_strides.size(); ++d) dst.t.strides[d] = l.view_strides[d];
      }
      rc = fluidml_hip_attention(&a.t, &kt.t, &v.t, &dst.t, l.s0, l.divisor ? 1 : 0, l.has_mask ? &mask.t : nullptr,
                                 l.has_cond ? &cond.t : nullptr, l.s1, ctx.stream);
      break;
    }
    case Launch::Kind::AddLayerNorm: {
      const kernel::TensorView b = ViewOf(Resolve(l.b), l.b);
      const kernel::Kernel &ln = *steps_[l.owner].kernel;
      const kernel::DeviceConstant *scale = ln.GetConstant(0), *bias = ln.GetConstant(1);
      if (scale == nullptr || bias == nullptr) throw std::logic_error("fused LayerNorm: the node holds no scale/bias");
      const kernel::TensorView g = scale->View(), h = bias->View();
      rc = fluidml_hip_add_layer_normalization(&a.t, &b.t, &g.t, &h.t, &out.t, l.axis, l.s0, ctx.stream);
      break;
    }
    case Launch::Kind::GatherStats: {
      const kernel::DeviceConstant *table = steps_[l.owner].kernel->GetConstant(0);
      if (table == nullptr) throw std::logic_error("Gather with statistics: the node holds no data tensor");
      const kernel::TensorView data = table->View();
      rc = fluidml_hip_gather_constant_data_tensor_stats(&a.t, &data.t, &out.t,
                                                         static_cast<float *>(privates_.at(l.norm_stats_out).device),
                                                         ctx.stream);
      break;
    }
    case Launch::Kind::GatherAddLayerNorm: {
      const kernel::DeviceConstant *table = steps_[l.owner].kernel->GetConstant(0);
      const kernel::DeviceConstant *table2 = l.has_gate ? steps_[l.owner2].kernel->GetConstant(0) : nullptr;
      const kernel::Kernel &ln = *steps_[l.norm_owner].kernel;
      const kernel::DeviceConstant *scale = ln.GetConstant(0), *bias = ln.GetConstant(1);
      if (table == nullptr || (l.has_gate && table2 == nullptr) || scale == nullptr || bias == nullptr) {
        throw std::logic_error("fused embedding: a node holds no table / scale / bias");
      }
      const kernel::TensorView data = table->View(), b = ViewOf(Resolve(l.b), l.b), c = ViewOf(Resolve(l.c), l.c);
      const kernel::TensorView g = scale->View(), h = bias->View();
      if (l.has_gate) {
        const kernel::TensorView data2 = table2->View();
        rc = fluidml_hip_gather_add_layer_normalization(&a.t, &data.t, &b.t, &data2.t, &c.t, &g.t, &h.t, &out.t, l.s0, ctx.stream);
      } else {
        rc = fluidml_hip_gather_add_layer_normalization(&a.t, &data.t, nullptr, &b.t, &c.t, &g.t, &h.t, &out.t, l.s0, ctx.stream);
      }
      break;
    }
    case Launch::Kind::CopyInto:
      rc = fluidml_hip_reshape(&a.t, &out.t, ctx.stream);  // same shape on both sides: a strided copy
      break;
    case Launch::Kind::PadViewCopy: {
      const Step &pad = steps_[l.members.front()];
      std::vector<int64_t> before, padded(pad.out.meta.GetShape());
      for (const auto &pr : pad.node->GetAttrs().pad_pairs) before.push_back(std::get<0>(pr));
      rc = fluidml_hip_pad_view_copy(&a.t, before.data(), padded.data(), static_cast<int32_t>(before.size()), l.view_offset,
                                     l.view_strides.data(), &out.t, ctx.stream);
      break;
    }
    case Launch::Kind::ReshapeTranspose: {
      // the Transpose's output buffer addressed by the Reshape's logical index
      const fl_tensor dst = Permuted(out.t, l.perm, true);
      rc = fluidml_hip_reshape(&a.t, &dst, ctx.stream);
      break;
    }
    case Launch::Kind::TransposeReshape: {
      // the Transpose's input buffer addressed by the Transpose's logical output index
      const fl_tensor src = Permuted(a.t, l.perm, false);
      rc = fluidml_hip_reshape(&src, &out.t, ctx.stream);
      break;
    }
    default: break;
  }
  if (rc_out != nullptr) {
    *rc_out = rc;
    return;
  }
  if (rc != 0) {
    ctx.Note(rc, LaunchKindName(l.kind));
    std::string what = std::string("launching fused ") + LaunchKindName(l.kind) + " of " + std::to_string(l.members.size()) +
                       " steps ending at node '" + steps_[l.members.back()].node->GetName() + "'";
    if (l.norm_mode != 0) what += " (deferred LayerNormalization, form " + std::to_string(l.norm_mode) + ")";
    if (!l.norm_stats_out.empty()) what += " (writes row statistics)";
    throw std::runtime_error(what + ": " + fluidml_hip_error_string(rc));
  }
}

void LaunchPlan::LaunchAll(kernel::LaunchContext &ctx) const {
  const std::vector<Launch> &schedule = GetSchedule();
  if (regions_.empty() || side_stream_ == nullptr) {
    for (const Launch &l : schedule) Issue(ctx, l);
    return;
  }
  kernel::LaunchContext side = ctx;
  side.stream = side_stream_;
  size_t r = 0;
  for (size_t i = 0; i < schedule.size(); ++i) {
    const bool inside = r < regions_.size() && i >= regions_[r].a_begin;
    if (inside && i == regions_[r].a_begin) {
      // fork: the second stream starts from the state the plan's stream has reached
      Check(fluidml_hip_event_record(region_events_[2 * r], ctx.stream), "recording a fork");
      Check(fluidml_hip_stream_wait_event(side_stream_, region_events_[2 * r]), "forking the second stream");
    }
    if (inside && i >= regions_[r].b_begin) {
      Issue(side, schedule[i]);
    } else {
      Issue(ctx, schedule[i]);
    }
    if (inside && i + 1 == regions_[r].end) {
      Check(fluidml_hip_event_record(region_events_[2 * r + 1], side_stream_), "recording a join");
      Check(fluidml_hip_stream_wait_event(ctx.stream, region_events_[2 * r + 1]), "joining the second stream");
      ++r;
    }
  }
  if (side.status != 0 && ctx.status == 0) {
    ctx.status = side.status;
    ctx.failed = side.failed;
  }
}

// One replay of the whole sequence on the plan's stream: the captured graph
// when capture is enabled (recorded on first use), plain launches otherwise.
void LaunchPlan::Replay(kernel::LaunchContext &ctx) {
  if (!use_graph_) {
    LaunchAll(ctx);
    return;
  }
  if (graph_ == nullptr) {
    Check(fluidml_hip_graph_begin_capture(stream_), "starting launch-plan capture");
    try {
      LaunchAll(ctx);
    } catch (...) {
      void *discard = nullptr;
      fluidml_hip_graph_end_capture(stream_, &discard);
      if (discard) fluidml_hip_graph_destroy(discard);
      throw;
    }
    Check(fluidml_hip_graph_end_capture(stream_, &graph_), "finishing launch-plan capture");
  }
  Check(fluidml_hip_graph_launch(graph_, stream_), "launching the captured plan");
}

size_t LaunchPlan::Run(const std::unordered_map<std::string, void *> &args, size_t epoch) {
  if (epoch == 0) epoch = 1;
  Materialize();
  // the literal LayerNorm mode reads its scratch before writing it: give every
  // call the zero-filled arena the reference allocates per Invoke (runner.cpp:87-88)
  if (flags_ & FL_REF_LN_STALE_SCRATCH) Check(fluidml_hip_arena_zero(arena_, arena_bytes_, stream_), "zeroing the arena");
  for (const Argument &a : arguments_) {
    void *host = args.at(a.name);
    if (a.type == Argument::Type::Input) {
      Check(fluidml_hip_memcpy_h2d(interfaces_.at(a.name).device, host, a.meta.GetSize(), stream_), "copying an input to HBM");
    }
  }
  Check(fluidml_hip_stream_synchronize(stream_), "waiting for input copies");
  DecideBranches();
  kernel::LaunchContext ctx;
  ctx.stream = stream_;
  ctx.flags = flags_;
  ctx.bf16 = bf16_;
  if (use_graph_ && graph_ == nullptr) {  // record outside the timed region
    Replay(ctx);
    Check(fluidml_hip_stream_synchronize(stream_), "waiting for the first replay");
  }
  const auto t0 = std::chrono::high_resolution_clock::now();
  for (size_t e = 0; e < epoch; ++e) Replay(ctx);
  Check(fluidml_hip_stream_synchronize(stream_), "waiting for the replays");
  const auto t1 = std::chrono::high_resolution_clock::now();
  for (const Argument &a : arguments_) {
    if (a.type == Argument::Type::Output) {
      Check(fluidml_hip_memcpy_d2h(args.at(a.name), interfaces_.at(a.name).device, a.meta.GetSize(), stream_), "copying an output to the host");
    }
  }
  Check(fluidml_hip_stream_synchronize(stream_), "waiting for output copies");
  return static_cast<size_t>(std::chrono::duration_cast<std::chrono::nanoseconds>(t1 - t0).count()) / epoch;
}

// Which kernels gain from running beside each other is not something the estimate above can tell (GPT-NeoX: its MLP
// beside the attention block gains nothing, the next layer's first projections beside an attention block 12 us;
// ConvBERT loses with every region), so the schedule with its regions and the one without them are both replayed on
// the first inputs and the faster one stays.
void LaunchPlan::DecideBranches() {
  if (branches_decided_) return;
  branches_decided_ = true;
  had_regions_ = !regions_.empty();
  const char *env = std::getenv("FLUIDML_BRANCH_CHECK");
  const bool env_check = env == nullptr || std::strtol(env, nullptr, 10) != 0;
  if (regions_.empty() || (branch_decision_ < 0 && (!branch_check_ || !env_check))) return;
  auto rebuild = [&](bool off) {
    Check(fluidml_hip_stream_synchronize(stream_), "waiting for the timed replays");
    if (graph_ != nullptr) {
      fluidml_hip_graph_destroy(graph_);
      graph_ = nullptr;
    }
    branches_off_ = off;
    schedule_built_ = false;
    GetSchedule();
    ApplyContractionPicks();
  };
  if (branch_decision_ >= 0) {
    // the decision of an earlier compile, read back from its JSON: nothing is timed
    if (branch_decision_ == 0) rebuild(true);
  } else {
    const double with = TimeReplayNs(2, 12);
    rebuild(true);
    const double without = TimeReplayNs(2, 12);
    if (with < 0.985 * without) rebuild(false);  // (the same regions and the same buffers again: planning is deterministic)
  }
  if (branches_off_) {
    // nothing writes the side branches' buffers any more
    for (auto it = privates_.begin(); it != privates_.end();) {
      if (it->first.compare(0, 5, "side:") == 0) {
        fluidml_hip_free(it->second.device);
        it = privates_.erase(it);
      } else {
        ++it;
      }
    }
  }
}

// ---- tile configurations of the contraction launches ----------------------------------------------------------

namespace {
bool IsContractionStep(const Step &s) {
  const flow::OpKind k = s.node->GetKind();
  return k == flow::OpKind::MatMul || k == flow::OpKind::GemmConstantWeightsBias;
}

void OperandSignature(std::ostream &os, const Operand &op) {
  const std::vector<int64_t> &shape = op.meta.GetShape();
  os << "[";
  for (size_t i = 0; i < shape.size(); ++i) os << (i ? "," : "") << shape[i];
  os << "]";
  int64_t first_byte = 0;
  if (op.viewed) {
    os << "v(";
    for (size_t i = 0; i < op.view_strides.size(); ++i) os << (i ? "," : "") << op.view_strides[i];
    os << ")";
    first_byte = op.view_offset * static_cast<int64_t>(GetSize(op.meta.GetType()));
  } else {
    os << "l(";
    for (size_t i = 0; i < op.layout.size(); ++i) os << (i ? "," : "") << op.layout[i];
    os << ")";
  }
  // arena and pooled private tensors sit at byte offsets of the memory plan inside 256-byte aligned allocations;
  // everything else is an allocation of its own
  if (op.space == Operand::Space::Arena || (op.space == Operand::Space::Private && !op.pool.empty())) {
    first_byte += static_cast<int64_t>(op.offset);
  }
  os << (first_byte % 16 == 0 ? "a" : "u");
}
}  // namespace

std::string LaunchPlan::ContractionSignature(size_t i) const {
  const Launch &l = GetSchedule().at(i);
  std::ostringstream os;
  auto chain_tag = [&](const Launch &x) {
    os << " b" << (x.has_c ? 1 : 0) << "c" << x.chain.n << "s" << (x.has_skip ? (x.has_skip2 ? 2 : 1) : 0);
    if (x.norm_mode != 0 || !x.norm_stats_out.empty()) os << " norm" << x.norm_mode << (x.norm_stats_out.empty() ? "" : "e");
    if (!x.view_strides.empty()) {
      os << " view(";
      for (size_t d = 0; d < x.view_strides.size(); ++d) os << (d ? "," : "") << x.view_strides[d];
      os << ")i" << x.n_inner << "o" << x.stride_outer;
    }
  };
  switch (l.kind) {
    case Launch::Kind::Step: {
      const Step &s = steps_[l.members[0]];
      if (!IsContractionStep(s)) return std::string();
      os << s.kernel->GetKernelName() << " ";
      OperandSignature(os, l.rewired ? l.a : s.in0);
      os << "x";
      OperandSignature(os, l.rewired ? l.b : s.in1);
      os << "->";
      OperandSignature(os, l.rewired ? l.out : s.out);
      const flow::Attrs &at = s.node->GetAttrs();
      os << " ta" << (at.trans_a ? 1 : 0) << "tb" << (at.trans_b ? 1 : 0);
      break;
    }
    case Launch::Kind::MatMulChain:
    case Launch::Kind::GemmChain: {
      os << LaunchKindName(l.kind) << " ";
      OperandSignature(os, l.a);
      os << "x";
      OperandSignature(os, l.b);
      os << "->";
      OperandSignature(os, l.out);
      chain_tag(l);
      if (l.kind == Launch::Kind::GemmChain) {
        const flow::Attrs &at = steps_[l.owner].node->GetAttrs();
        os << " ta" << (at.trans_a ? 1 : 0) << "tb" << (at.trans_b ? 1 : 0);
      }
      break;
    }
    case Launch::Kind::MatMulGroup: {
      os << LaunchKindName(l.kind) << " ";
      OperandSignature(os, l.a);
      if (l.norm_mode != 0) os << " norm" << l.norm_mode;
      for (const Launch &m : l.group) {
        os << " x";
        OperandSignature(os, m.b);
        os << "->";
        OperandSignature(os, m.out);
        chain_tag(m);
      }
      break;
    }
    default: return std::string();
  }
  if (bf16_) os << " bf16";
  return os.str();
}

void LaunchPlan::ApplyContractionPicks() const {
  const std::vector<Launch> &schedule = GetSchedule();
  for (size_t i = 0; i < schedule.size(); ++i) {
    schedule_[i].contract = 0;
    if (table_ == nullptr || table_->GetMode() == kernel::ContractionTable::Mode::Off) continue;
    const std::string signature = ContractionSignature(i);
    kernel::ContractPick pick;
    if (!signature.empty() && table_->Find(signature, &pick)) schedule_[i].contract = pick.Flags();
  }
}

std::vector<std::pair<std::string, uint32_t>> LaunchPlan::GetContractionChoices() const {
  std::vector<std::pair<std::string, uint32_t>> out;
  const std::vector<Launch> &schedule = GetSchedule();
  for (size_t i = 0; i < schedule.size(); ++i) {
    const std::string signature = ContractionSignature(i);
    if (!signature.empty()) out.push_back({signature, schedule[i].contract});
  }
  return out;
}

// Times the tile configurations of every contraction signature the table does not hold yet, inside this plan's
// own schedule: for each candidate the whole schedule is issued launch by launch with that candidate on all those
// contractions, so each one is timed with the operands, the cache state and the weights it really meets (timed
// alone in a loop, a projection's weights stay in the last-level cache; in the schedule every launch streams its
// own from HBM).  Durations are the dispatches' own begin/end timestamps.
void LaunchPlan::TuneContractions() {
  if (table_ == nullptr || table_->GetMode() == kernel::ContractionTable::Mode::Off) return;
  const std::vector<Launch> &schedule = GetSchedule();
  std::map<std::string, std::vector<size_t>> unknown;
  for (size_t i = 0; i < schedule.size(); ++i) {
    const std::string signature = ContractionSignature(i);
    if (!signature.empty() && !table_->Find(signature, nullptr)) unknown[signature].push_back(i);
  }
  if (!unknown.empty() && table_->GetMode() == kernel::ContractionTable::Mode::Measure) {
    std::vector<size_t> probes;
    for (const auto &kv : unknown) probes.insert(probes.end(), kv.second.begin(), kv.second.end());
    std::sort(probes.begin(), probes.end());
    std::vector<void *> events(2 * probes.size(), nullptr);
    for (void *&e : events) Check(fluidml_hip_event_create(&e), "event");
    kernel::LaunchContext ctx;
    ctx.stream = stream_;
    ctx.flags = flags_;
    ctx.bf16 = bf16_;
    constexpr int kRounds = 3;
    // durations[launch] of one candidate: the best of kRounds passes after one that warms up; false: refused
    auto time_candidate = [&](uint32_t bits, std::vector<double> *ns, std::vector<bool> *accepted) {
      ns->assign(probes.size(), std::numeric_limits<double>::max());
      accepted->assign(probes.size(), true);
      for (int round = 0; round <= kRounds; ++round) {
        size_t p = 0;
        for (size_t i = 0; i < schedule.size(); ++i) {
          if (p < probes.size() && probes[p] == i) {
            Launch probe = schedule[i];
            probe.contract = bits;
            int rc = 0;
            if ((*accepted)[p]) {
              Check(fluidml_hip_time_kernels(events[2 * p], events[2 * p + 1]), "kernel timing on");
              Issue(ctx, probe, &rc);
              Check(fluidml_hip_time_kernels(nullptr, nullptr), "kernel timing off");
              if (rc == FL_ERR_UNSUPPORTED) (*accepted)[p] = false;
              else if (rc != 0) Check(rc, "timing a contraction launch");
            }
            if (!(*accepted)[p]) {
              probe.contract = 0;  // keeps the tensors behind it defined
              Issue(ctx, probe);
            }
            ++p;
          } else {
            Issue(ctx, schedule[i]);
          }
        }
        Check(fluidml_hip_stream_synchronize(stream_), "tuning sync");
        if (round == 0) continue;
        for (size_t q = 0; q < probes.size(); ++q) {
          if (!(*accepted)[q]) continue;
          double t = 0;
          Check(fluidml_hip_event_elapsed_ns(events[2 * q], events[2 * q + 1], &t), "event elapsed");
          (*ns)[q] = std::min((*ns)[q], t);
        }
      }
    };
    try {
      std::map<size_t, size_t> probe_of;
      for (size_t q = 0; q < probes.size(); ++q) probe_of[probes[q]] = q;
      // total over a signature's launches, or a negative number if any of them refused the candidate
      auto total = [&](const std::vector<size_t> &launches, const std::vector<double> &ns, const std::vector<bool> &ok) {
        double sum = 0;
        for (size_t i : launches) {
          const size_t q = probe_of.at(i);
          if (!ok[q]) return -1.0;
          sum += ns[q];
        }
        return sum / static_cast<double>(launches.size());
      };
      std::vector<double> ns;
      std::vector<bool> ok;
      time_candidate(0, &ns, &ok);
      std::map<std::string, kernel::ContractPick> best;
      for (const auto &kv : unknown) {
        kernel::ContractPick rule;
        rule.ns = rule.rule_ns = total(kv.second, ns, ok);
        if (rule.ns < 0) throw std::runtime_error("tuning: the library's rule refused '" + kv.first + "'");
        best[kv.first] = rule;
      }
      for (const auto &c : kernel::ContractionTable::Candidates(true)) {
        kernel::ContractPick cand;
        cand.tile = c.first;
        cand.splits = c.second;
        time_candidate(cand.Flags(), &ns, &ok);
        for (const auto &kv : unknown) {
          kernel::ContractPick &b = best[kv.first];
          cand.ns = total(kv.second, ns, ok);
          cand.rule_ns = b.rule_ns;
          if (cand.ns < 0) continue;
          const double bar = b.IsRule() ? b.rule_ns * (1.0 - kernel::kTuneMargin) : b.ns;
          if (cand.ns < bar) b = cand;
        }
      }
      for (const auto &kv : best) table_->Put(kv.first, kv.second);
    } catch (...) {
      fluidml_hip_time_kernels(nullptr, nullptr);
      for (void *e : events) fluidml_hip_event_destroy(e);
      throw;
    }
    for (void *e : events) fluidml_hip_event_destroy(e);
  }
  ApplyContractionPicks();
}

void LaunchPlan::Settle() {
  Materialize();
  DecideBranches();
}

void LaunchPlan::ReplayResident(size_t n) {
  Materialize();
  DecideBranches();
  kernel::LaunchContext ctx;
  ctx.stream = stream_;
  ctx.flags = flags_;
  ctx.bf16 = bf16_;
  for (size_t i = 0; i < n; ++i) Replay(ctx);
  Check(fluidml_hip_stream_synchronize(stream_), "waiting for the replays");
}

double LaunchPlan::TimeReplayNs(size_t warmup, size_t iters) {
  Materialize();
  DecideBranches();
  kernel::LaunchContext ctx;
  ctx.stream = stream_;
  ctx.flags = flags_;
  ctx.bf16 = bf16_;
  for (size_t i = 0; i < warmup + 1; ++i) Replay(ctx);
  void *e0 = nullptr, *e1 = nullptr;
  Check(fluidml_hip_event_create(&e0), "event");
  Check(fluidml_hip_event_create(&e1), "event");
  Check(fluidml_hip_event_record(e0, stream_), "event record");
  for (size_t i = 0; i < iters; ++i) Replay(ctx);
  Check(fluidml_hip_event_record(e1, stream_), "event record");
  double ns = 0;
  Check(fluidml_hip_event_elapsed_ns(e0, e1, &ns), "event elapsed");
  fluidml_hip_event_destroy(e0);
  fluidml_hip_event_destroy(e1);
  return ns / static_cast<double>(std::max<size_t>(iters, 1));
}

std::vector<double> LaunchPlan::ReplayTimesNs(size_t warmup, size_t iters) {
  Materialize();
  DecideBranches();
  kernel::LaunchContext ctx;
  ctx.stream = stream_;
  ctx.flags = flags_;
  ctx.bf16 = bf16_;
  for (size_t i = 0; i < warmup + 1; ++i) Replay(ctx);
  std::vector<void *> events(iters + 1, nullptr);
  for (void *&e : events) Check(fluidml_hip_event_create(&e), "event");
  Check(fluidml_hip_event_record(events[0], stream_), "event record");
  for (size_t i = 0; i < iters; ++i) {
    Replay(ctx);
    Check(fluidml_hip_event_record(events[i + 1], stream_), "event record");
  }
  Check(fluidml_hip_stream_synchronize(stream_), "waiting for the replays");
  std::vector<double> out(iters, 0.0);
  for (size_t i = 0; i < iters; ++i) Check(fluidml_hip_event_elapsed_ns(events[i], events[i + 1], &out[i]), "event elapsed");
  for (void *e : events) fluidml_hip_event_destroy(e);
  return out;
}

std::vector<StepTime> LaunchPlan::Profile(size_t warmup, size_t iters) {
  Materialize();
  DecideBranches();
  kernel::LaunchContext ctx;
  ctx.stream = stream_;
  ctx.flags = flags_;
  ctx.bf16 = bf16_;
  const std::vector<Launch> &schedule = GetSchedule();
  std::vector<std::vector<double>> samples(schedule.size());
  // one start/stop pair per launch, stamped by the dispatch itself (kernel-exact durations)
  std::vector<void *> events(2 * schedule.size(), nullptr);
  for (void *&e : events) Check(fluidml_hip_event_create(&e), "event");
  for (size_t it = 0; it < warmup + iters; ++it) {
    try {
      for (size_t i = 0; i < schedule.size(); ++i) {
        if (schedule[i].kind == Launch::Kind::View || schedule[i].kind == Launch::Kind::Placed) continue;
        Check(fluidml_hip_time_kernels(events[2 * i], events[2 * i + 1]), "kernel timing on");
        Issue(ctx, schedule[i]);
      }
    } catch (...) {
      fluidml_hip_time_kernels(nullptr, nullptr);
      throw;
    }
    Check(fluidml_hip_time_kernels(nullptr, nullptr), "kernel timing off");
    Check(fluidml_hip_stream_synchronize(stream_), "profiling sync");
    if (it >= warmup) {
      for (size_t i = 0; i < schedule.size(); ++i) {
        if (schedule[i].kind == Launch::Kind::View || schedule[i].kind == Launch::Kind::Placed) continue;
        double ns = 0;
        Check(fluidml_hip_event_elapsed_ns(events[2 * i], events[2 * i + 1], &ns), "event elapsed");
        samples[i].push_back(ns);
      }
    }
  }
  for (void *e : events) fluidml_hip_event_destroy(e);
  std::vector<StepTime> out;
  for (size_t i = 0; i < schedule.size(); ++i) {
    std::vector<double> &v = samples[i];
    std::sort(v.begin(), v.end());
    const Launch &l = schedule[i];
    if (l.kind == Launch::Kind::View || l.kind == Launch::Kind::Placed) continue;  // not a launch
    StepTime t;
    for (size_t m : l.members) {
      t.node += (t.node.empty() ? "" : "+") + steps_[m].node->GetName();
      t.kernel += (t.kernel.empty() ? "" : "+") + steps_[m].kernel->GetKernelName();
    }
    t.ns = v.empty() ? 0 : v[v.size() / 2];
    t.bytes = l.bytes;
    t.flops = l.flops;
    out.push_back(std::move(t));
  }
  return out;
}

}  // namespace worker
}  // namespace fluidml
