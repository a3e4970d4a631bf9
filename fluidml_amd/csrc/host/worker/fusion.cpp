// Launch-level fusion: groups the steps of a launch plan into chains that one
// HIP kernel computes.  The node sequence, the memory plan and every tensor a
// later step (or the caller) can observe stay exactly as planned; only tensors
// with a single reader inside a chain are no longer written.  The reference
// fuses at graph level before planning (e.g. its AddDivErfAddMulMul node,
// src/structure/flow/node.cpp); it has no counterpart of this pass because it
// pays no per-kernel launch cost.
#include <algorithm>
#include <cstdlib>
#include <optional>
#include <string>
#include <unordered_map>

#include "utils/utils.h"
#include "worker/launcher.h"

namespace fluidml {
namespace worker {

const char *LaunchKindName(Launch::Kind kind) {
  switch (kind) {
    case Launch::Kind::Step: return "Step";
    case Launch::Kind::MatMulChain: return "MatMulChain";
    case Launch::Kind::MatMulGroup: return "MatMulGroup";
    case Launch::Kind::GemmChain: return "GemmChain";
    case Launch::Kind::ConvChain: return "ConvChain";
    case Launch::Kind::PadViewCopy: return "PadViewCopy";
    case Launch::Kind::ConvPair: return "ConvPair";
    case Launch::Kind::SoftmaxMatVec: return "SoftmaxMatVec";
    case Launch::Kind::ElementwiseChain: return "ElementwiseChain";
    case Launch::Kind::MulAdd: return "MulAdd";
    case Launch::Kind::AddAdd: return "AddAdd";
    case Launch::Kind::GatherAdd: return "GatherAdd";
    case Launch::Kind::Rotary: return "Rotary";
    case Launch::Kind::RotaryPair: return "RotaryPair";
    case Launch::Kind::DivAddSoftmax: return "DivAddSoftmax";
    case Launch::Kind::Attention: return "Attention";
    case Launch::Kind::AddLayerNorm: return "AddLayerNormalization";
    case Launch::Kind::GatherAddLayerNorm: return "GatherAddLayerNormalization";
    case Launch::Kind::GatherStats: return "GatherStatistics";
    case Launch::Kind::ReshapeTranspose: return "ReshapeTranspose";
    case Launch::Kind::View: return "View";
    case Launch::Kind::Placed: return "Placed";
    case Launch::Kind::CopyInto: return "CopyInto";
    default: return "TransposeReshape";
  }
}

namespace {

using flow::OpKind;

bool SameTensor(const Operand &x, const Operand &y) { return x.space == y.space && x.name == y.name; }

// an intermediate may be elided only if nobody outside the plan can see it
bool Elidable(const Operand &o) { return o.space == Operand::Space::Arena || o.space == Operand::Space::Private; }

bool Alias(const Operand &x, const Operand &y) {
  if (x.space != y.space) return false;
  if (x.space != Operand::Space::Arena) return x.name == y.name;
  const size_t x1 = x.offset + x.Extent(), y1 = y.offset + y.Extent();
  return x.offset < y1 && y.offset < x1;
}

bool IsFloat(const Operand &o) { return o.meta.GetType() == Type::kFloat32; }

// Follows a tensor through Reshape / Transpose steps and answers whether the result is just the source tensor
// re-addressed.  Every source dim is kept as a run of "atoms" (factors of its extent, outermost first); a reshape
// regroups the row-major sequence of atoms and may cut one in two, a transpose permutes groups.
class ViewTracker {
 public:
  explicit ViewTracker(const std::vector<int64_t> &source_shape) {
    for (size_t d = 0; d < source_shape.size(); ++d) {
      atoms_.push_back({static_cast<int>(d), source_shape[d]});
      dims_.push_back({static_cast<int>(atoms_.size()) - 1});
    }
    n_source_dims_ = source_shape.size();
  }

  // row-major reshape to `shape`; false (state unusable) if an atom would have to be cut unevenly
  bool Reshape(const std::vector<int64_t> &shape) {
    std::vector<int> flat;
    for (const auto &d : dims_) flat.insert(flat.end(), d.begin(), d.end());
    std::vector<std::vector<int>> out;
    size_t pos = 0;
    for (int64_t extent : shape) {
      std::vector<int> group;
      int64_t need = extent;
      while (need > 1) {
        if (pos >= flat.size()) return false;
        const int a = flat[pos];
        const int64_t e = atoms_[a].extent;
        if (e == 1) {
          ++pos;
        } else if (need % e == 0) {
          group.push_back(a);
          need /= e;
          ++pos;
        } else if (e % need == 0) {
          // the outer part of the atom completes this dim, the inner part stays for the next one
          atoms_.push_back({atoms_[a].source_dim, e / need});
          const int inner = static_cast<int>(atoms_.size()) - 1;
          atoms_[a].extent = need;
          if (auto it = inner_of_.find(a); it != inner_of_.end()) inner_of_[inner] = it->second;
          inner_of_[a] = inner;
          group.push_back(a);
          flat[pos] = inner;
          need = 1;
        } else {
          return false;
        }
      }
      out.push_back(std::move(group));
    }
    for (; pos < flat.size(); ++pos) {
      if (atoms_[flat[pos]].extent != 1) return false;
    }
    dims_ = std::move(out);
    return true;
  }

  bool Transpose(const std::vector<int64_t> &perm) {
    if (perm.size() != dims_.size()) return false;
    std::vector<std::vector<int>> out;
    for (int64_t p : perm) {
      if (p < 0 || static_cast<size_t>(p) >= dims_.size()) return false;
      out.push_back(dims_[static_cast<size_t>(p)]);
    }
    dims_ = std::move(out);
    return true;
  }

  struct View {
    std::vector<int64_t> strides;  // per source dim
    int64_t n_inner = 0, stride_outer = 0;  // split of the one source dim that may be split, if any
  };

  // Strides of the source dims inside a tensor of the current shape stored with `strides`.  Every source dim
  // must come out as one stride, except one (`split_dim`; negative: the last) which may be two (outer, inner).
  std::optional<View> Resolve(const std::vector<int64_t> &strides, int split_dim = -1) const {
    const size_t may_split = split_dim < 0 ? n_source_dims_ - 1 : static_cast<size_t>(split_dim);
    if (strides.size() != dims_.size()) return std::nullopt;
    std::vector<int64_t> atom_stride(atoms_.size(), 0);
    for (size_t d = 0; d < dims_.size(); ++d) {
      int64_t run = strides[d];
      for (size_t k = dims_[d].size(); k-- > 0;) {
        atom_stride[dims_[d][k]] = run;
        run *= atoms_[dims_[d][k]].extent;
      }
    }
    View v;
    v.strides.assign(n_source_dims_, 0);
    for (size_t d = 0; d < n_source_dims_; ++d) {
      // atoms of this source dim, outermost first, merged where contiguous, unit extents dropped
      std::vector<std::pair<int64_t, int64_t>> parts;  // (extent, stride)
      for (int a = static_cast<int>(d); a >= 0;) {
        if (atoms_[a].extent != 1) {
          if (!parts.empty() && parts.back().second == atom_stride[a] * atoms_[a].extent) {
            parts.back().first *= atoms_[a].extent;
            parts.back().second = atom_stride[a];
          } else {
            parts.push_back({atoms_[a].extent, atom_stride[a]});
          }
        }
        auto it = inner_of_.find(a);
        a = it == inner_of_.end() ? -1 : it->second;
      }
      if (parts.empty()) continue;
      if (parts.size() == 1) {
        v.strides[d] = parts[0].second;
      } else if (parts.size() == 2 && d == may_split) {
        v.stride_outer = parts[0].second;
        v.n_inner = parts[1].first;
        v.strides[d] = parts[1].second;
      } else {
        return std::nullopt;
      }
    }
    return v;
  }

  // The other direction: element strides of the current dims inside the source tensor stored with
  // `source_strides`; nullopt if a current dim is not one strided run of the source.
  std::optional<std::vector<int64_t>> StridesInSource(const std::vector<int64_t> &source_strides) const {
    if (source_strides.size() != n_source_dims_) return std::nullopt;
    std::vector<int64_t> atom_stride(atoms_.size(), 0);
    for (size_t d = 0; d < n_source_dims_; ++d) {
      std::vector<int> chain;  // atoms of source dim d, outermost first
      for (int a = static_cast<int>(d); a >= 0;) {
        chain.push_back(a);
        auto it = inner_of_.find(a);
        a = it == inner_of_.end() ? -1 : it->second;
      }
      int64_t run = source_strides[d];
      for (size_t k = chain.size(); k-- > 0;) {
        atom_stride[chain[k]] = run;
        run *= atoms_[chain[k]].extent;
      }
    }
    std::vector<int64_t> out;
    for (const auto &dim : dims_) {
      int64_t stride = 0;
      for (size_t k = 0; k < dim.size(); ++k) {
        if (k + 1 < dim.size() && atom_stride[dim[k]] != atom_stride[dim[k + 1]] * atoms_[dim[k + 1]].extent) return std::nullopt;
        stride = atom_stride[dim[k]];
      }
      out.push_back(stride);  // 0 for a unit dim
    }
    return out;
  }

 private:
  struct Atom {
    int source_dim;
    int64_t extent;
  };
  std::vector<Atom> atoms_;                  // atoms 0..n_source_dims-1 are the outermost atom of each source dim
  std::unordered_map<int, int> inner_of_;    // atom -> the atom cut off its inner side
  std::vector<std::vector<int>> dims_;       // current dims, each a run of atoms (outermost first)
  size_t n_source_dims_ = 0;
};

class Scheduler {
 public:
  Scheduler(const std::vector<Step> &steps)
      : steps_(steps), taken_(steps.size(), false), elided_(steps.size(), false), rewired_(steps.size(), false),
        placed_(steps.size(), 0), filled_(steps.size(), false) {
    BuildReaders();
  }

  std::vector<Launch> Run(bool fuse) {
    std::vector<Launch> fused;
    if (fuse) {
      // the row-reduction patterns first: their leading Div/Add would otherwise be absorbed one at a time
      // by the elementwise chains of the second sweep, which saves fewer launches
      for (size_t i = 0; i < steps_.size(); ++i) {
        if (taken_[i]) continue;
        std::optional<Launch> l;
        if (Kind(i) == OpKind::MatMul) l = MatchAttention(i);
        else if (Kind(i) == OpKind::DivConstantRhs) l = MatchSoftmax(i);
        else if (Kind(i) == OpKind::AddCommon) l = MatchLayerNorm(i);
        if (!l && Kind(i) == OpKind::AddCommon) l = MatchRotary(i);
        if (l) {
          for (size_t m : l->members) taken_[m] = true;
          fused.push_back(std::move(*l));
        }
      }
      for (size_t i = 0; i < steps_.size(); ++i) {
        if (taken_[i]) continue;
        std::optional<Launch> l;
        switch (Kind(i)) {
          case OpKind::MatMul:
          case OpKind::GemmConstantWeightsBias:
          case OpKind::ConvWithPadding:
          case OpKind::ConvWithoutPadding:
            l = MatchConvPair(i);
            if (!l) l = MatchContraction(i);
            break;
          case OpKind::Softmax: l = MatchSoftmaxMatVec(i); break;
          case OpKind::MulCommon: l = MatchMulAdd(i); break;
          case OpKind::AddCommon: l = MatchAddAdd(i); break;
          case OpKind::GatherConstantDataTensor: l = MatchGatherAdd(i); break;
          case OpKind::Pad: l = MatchPadViewCopy(i); break;
          case OpKind::Reshape: l = MatchCopyPair(i, OpKind::Transpose); break;
          case OpKind::Transpose: l = MatchCopyPair(i, OpKind::Reshape); break;
          default: break;
        }
        if (!l && UnaryOp(i) >= 0) l = MatchElementwise(i);
        if (l) {
          for (size_t m : l->members) taken_[m] = true;
          fused.push_back(std::move(*l));
        }
      }
    }
    for (const std::string &name : pending_moves_) MoveOut(name, {&fused});
    pending_moves_.clear();
    if (fuse) {
      MarkSilent(fused);
      GroupSiblings(&fused);
      silent_.clear();
    }
    if (fuse) PlacePadInputs(&fused);
    if (fuse) ElideViews(&fused);
    if (fuse) RetryAttention(&fused);
    if (fuse) RetrySoftmaxMatVec(&fused);
    if (fuse) {
      MarkSilent(fused);
      PairRotary(&fused);
      silent_.clear();
    }
    if (fuse) DeferLayerNorms(&fused);
    if (fuse) FuseEmbeddings(&fused);
    if (fuse) PlaceConcatInputs(&fused);
    // a chain is issued where its last member stood; everything else keeps its place
    std::vector<const Launch *> at(steps_.size(), nullptr);
    for (const Launch &l : fused) at[l.kind == Launch::Kind::MatMulGroup ? l.position : l.members.back()] = &l;
    std::vector<Launch> schedule;
    for (size_t i = 0; i < steps_.size(); ++i) {
      if (at[i] != nullptr) {
        schedule.push_back(*at[i]);
      } else if (elided_[i]) {
        Launch l;
        l.kind = Launch::Kind::View;
        l.members = {i};
        l.out = steps_[i].out;  // rewritten: the source seen as this step's output
        schedule.push_back(std::move(l));
      } else if (filled_[i]) {
        // a Reshape whose input was written straight into its buffer
        Launch l;
        l.kind = Launch::Kind::Placed;
        l.members = {i};
        l.out = steps_[i].out;
        schedule.push_back(std::move(l));
      } else if (placed_[i] != 0) {
        // a Concat2 with one or both inputs already in place
        Launch l;
        l.members = {i};
        if (placed_[i] == 3) {
          l.kind = Launch::Kind::Placed;
          l.out = steps_[i].out;
        } else {
          l.kind = Launch::Kind::CopyInto;
          const bool first_left = placed_[i] == 2;  // input 1 is in place: copy input 0
          l.a = first_left ? steps_[i].in0 : steps_[i].in1;
          l.out = ConcatPart(i, first_left ? 0 : 1);
          l.bytes = 2.0 * static_cast<double>(l.a.meta.GetSize());
        }
        schedule.push_back(std::move(l));
      } else if (!taken_[i]) {
        Launch l;
        l.members = {i};
        l.bytes = steps_[i].bytes;
        l.flops = steps_[i].flops;
        if (rewired_[i]) {
          l.rewired = true;
          l.a = steps_[i].in0;
          l.b = steps_[i].in1;
          l.out = steps_[i].out;
        }
        schedule.push_back(std::move(l));
      }
    }
    return schedule;
  }

 private:
  void BuildReaders() {
    readers_.clear();
    producer_.clear();
    for (size_t i = 0; i < steps_.size(); ++i) {
      const Step &s = steps_[i];
      if (!s.out.viewed) producer_[s.out.name] = i;
      readers_[s.in0.name].push_back(i);
      if (s.node->IsDoubleInputs() && !SameTensor(s.in0, s.in1)) readers_[s.in1.name].push_back(i);
    }
  }

  // ---- tensors moved out of the arena ------------------------------------------------------------------
  // The memory plan gives every tensor its bytes for the span between its producer and its last reader in the
  // serial order, and reuses them outside it.  A fusion that makes a tensor appear earlier or be read later than
  // planned can therefore find other tenants on its bytes.  Such a tensor gets a buffer of its own outside the
  // arena instead (reported with the private bytes): the plan's offsets stay exactly the reference's, and the
  // fusion goes ahead.  Every operand copy that names the tensor is rewritten: the plan's steps (marked rewired,
  // so that single-step launches carry the operands too) and the operands held by the launches built so far.
  static bool MoveOperand(Operand *op, const std::string &name) {
    if (op->name != name || op->space != Operand::Space::Arena) return false;
    op->space = Operand::Space::Private;
    op->offset = 0;
    op->pool.clear();
    return true;
  }
  bool Movable(const Operand &op) const {
    if (op.space != Operand::Space::Arena || op.viewed || std::getenv("FLUIDML_MOVE_OUT_OFF") != nullptr) return false;
    const auto p = producer_.find(op.name);
    return p != producer_.end() && SameTensor(steps_[p->second].out, op);
  }
  // the tensor whose bytes `op` addresses: itself, or what the elided view(s) it is seen through look into
  std::optional<Operand> Underlying(const Operand &op) const {
    if (!op.viewed) return op;
    const auto p = producer_.find(op.name);
    if (p == producer_.end() || steps_[p->second].out.viewed || steps_[p->second].out.space != op.space) return std::nullopt;
    return steps_[p->second].out;
  }
  void MoveOut(const std::string &name, std::initializer_list<std::vector<Launch> *> lists) {
    for (size_t i = 0; i < steps_.size(); ++i) {
      Step &st = steps_[i];
      bool changed = MoveOperand(&st.in0, name);
      if (st.node->IsDoubleInputs()) changed = MoveOperand(&st.in1, name) || changed;
      changed = MoveOperand(&st.out, name) || changed;
      if (changed) rewired_[i] = true;
    }
    auto in_launch = [&](Launch &l) {
      for (Operand *op : {&l.a, &l.b, &l.c, &l.d, &l.e, &l.out, &l.out2}) MoveOperand(op, name);
    };
    for (std::vector<Launch> *list : lists) {
      for (Launch &l : *list) {
        in_launch(l);
        for (Launch &g : l.group) in_launch(g);
      }
    }
  }

  // ---- view elision -----------------------------------------------------------------------------------
  // A Slice, Transpose, Squeeze, Unsqueeze, a Gather whose constant indices form an arithmetic pattern (sliding
  // windows), or (where the result is still one strided pattern) a Reshape / Flatten that no fusion has absorbed
  // does not have to run: every kernel here takes element strides, so the readers
  // can address the step's input directly.  Allowed when the tensor is internal, and the bytes of the input stay
  // untouched from the step's position to the position where each reader is issued (the input may be dead in
  // the memory plan by then, and its bytes reused).

  static std::vector<int64_t> LogicalStrides(const Operand &op) {
    if (op.viewed) return op.view_strides;
    return utils::GenStrides(op.meta.GetShape(), op.layout);
  }

  // step i's output as a view of its input: (element offset, strides per output dim)
  std::optional<std::pair<int64_t, std::vector<int64_t>>> AsView(size_t i) const { return AsViewOf(i, steps_[i].in0); }

  // the same with the step's input taken to be `in0` (the step's own input, possibly seen through earlier views)
  std::optional<std::pair<int64_t, std::vector<int64_t>>> AsViewOf(size_t i, const Operand &in0) const {
    Step s = steps_[i];
    s.in0 = in0;
    const std::vector<int64_t> st = LogicalStrides(s.in0);
    const auto &ishape = s.in0.meta.GetShape();
    const auto &oshape = s.out.meta.GetShape();
    const int64_t irank = static_cast<int64_t>(ishape.size()), orank = static_cast<int64_t>(oshape.size());
    if (s.in0.meta.GetType() != s.out.meta.GetType()) return std::nullopt;
    int64_t offset = s.in0.viewed ? s.in0.view_offset : 0;
    std::vector<int64_t> strides;
    const flow::Attrs &at = Attrs(i);
    switch (Kind(i)) {
      case OpKind::Transpose: {
        if (irank != orank) return std::nullopt;
        std::vector<bool> seen(static_cast<size_t>(irank), false);
        for (int64_t k = 0; k < orank; ++k) {
          const int64_t p = at.perm.empty() ? irank - 1 - k : at.perm[static_cast<size_t>(k)];
          if (p < 0 || p >= irank || seen[static_cast<size_t>(p)] || oshape[static_cast<size_t>(k)] != ishape[static_cast<size_t>(p)]) return std::nullopt;
          seen[static_cast<size_t>(p)] = true;
          strides.push_back(st[static_cast<size_t>(p)]);
        }
        break;
      }
      case OpKind::Slice: {
        if (irank != orank || at.starts.size() != at.axes.size() || at.steps.size() != at.axes.size()) return std::nullopt;
        std::vector<int64_t> start(static_cast<size_t>(irank), 0), step(static_cast<size_t>(irank), 1);
        for (size_t n = 0; n < at.axes.size(); ++n) {
          int64_t ax = at.axes[n] < 0 ? at.axes[n] + irank : at.axes[n];
          if (ax < 0 || ax >= irank) return std::nullopt;
          int64_t b = at.starts[n];
          if (b < 0) b += ishape[static_cast<size_t>(ax)];
          if (b < 0 || at.steps[n] <= 0) return std::nullopt;
          start[static_cast<size_t>(ax)] = b;
          step[static_cast<size_t>(ax)] = at.steps[n];
        }
        for (size_t d = 0; d < static_cast<size_t>(irank); ++d) {
          if (start[d] + (oshape[d] - 1) * step[d] >= ishape[d]) return std::nullopt;
          offset += start[d] * st[d];
          strides.push_back(st[d] * step[d]);
        }
        break;
      }
      case OpKind::Squeeze: {
        if (irank != orank + static_cast<int64_t>(at.axes.size())) return std::nullopt;
        size_t j = 0;
        for (int64_t d = 0; d < irank; ++d) {
          bool squeezed = false;
          for (int64_t ax : at.axes) squeezed = squeezed || (ax < 0 ? ax + irank : ax) == d;
          if (squeezed) {
            if (ishape[static_cast<size_t>(d)] != 1) return std::nullopt;
          } else {
            if (j >= oshape.size() || oshape[j] != ishape[static_cast<size_t>(d)]) return std::nullopt;
            strides.push_back(st[static_cast<size_t>(d)]);
            ++j;
          }
        }
        if (j != oshape.size()) return std::nullopt;
        break;
      }
      case OpKind::Unsqueeze: {
        if (irank + static_cast<int64_t>(at.axes.size()) != orank) return std::nullopt;
        size_t j = 0;
        for (int64_t d = 0; d < orank; ++d) {
          bool added = false;
          for (int64_t ax : at.axes) added = added || (ax < 0 ? ax + orank : ax) == d;
          if (added) {
            if (oshape[static_cast<size_t>(d)] != 1) return std::nullopt;
            strides.push_back(0);
          } else {
            if (j >= ishape.size() || ishape[j] != oshape[static_cast<size_t>(d)]) return std::nullopt;
            strides.push_back(st[j++]);
          }
        }
        if (j != ishape.size()) return std::nullopt;
        break;
      }
      case OpKind::GatherConstantIndicesTensor: {
        // indices that form an arithmetic pattern, index[j0, j1, ..] = base + sum_d j_d * step_d with every step
        // >= 0 (the sliding windows of an unfolded convolution: index[s, k] = s + k), turn the gathered axis into
        // one strided dim per index dim; the windows may overlap, which a reader does not mind
        if (!at.t0) return std::nullopt;
        const Tensor &index = *at.t0;
        const auto &qshape = index.GetShape();
        const int64_t q = static_cast<int64_t>(qshape.size());
        int64_t axis = at.axis < 0 ? at.axis + irank : at.axis;
        if (axis < 0 || axis >= irank || orank != irank - 1 + q || q == 0) return std::nullopt;
        const std::vector<float64_t> &values = index.Get();
        int64_t count = 1;
        for (int64_t d : qshape) count *= d;
        if (count <= 0 || static_cast<int64_t>(values.size()) != count) return std::nullopt;
        const int64_t base = static_cast<int64_t>(values[0]);
        std::vector<int64_t> step(static_cast<size_t>(q), 0), unit(static_cast<size_t>(q), 1);
        for (int64_t d = q - 2; d >= 0; --d) unit[static_cast<size_t>(d)] = unit[static_cast<size_t>(d + 1)] * qshape[static_cast<size_t>(d + 1)];
        for (int64_t d = 0; d < q; ++d) {
          if (qshape[static_cast<size_t>(d)] > 1) step[static_cast<size_t>(d)] = static_cast<int64_t>(values[static_cast<size_t>(unit[static_cast<size_t>(d)])]) - base;
          if (step[static_cast<size_t>(d)] < 0) return std::nullopt;
        }
        for (int64_t n = 0; n < count; ++n) {
          int64_t rem = n, want = base;
          for (int64_t d = 0; d < q; ++d) {
            want += (rem / unit[static_cast<size_t>(d)]) * step[static_cast<size_t>(d)];
            rem %= unit[static_cast<size_t>(d)];
          }
          const int64_t have = static_cast<int64_t>(values[static_cast<size_t>(n)]);
          if (have != want || static_cast<float64_t>(have) != values[static_cast<size_t>(n)] || have < 0 ||
              have >= ishape[static_cast<size_t>(axis)]) {
            return std::nullopt;
          }
        }
        for (int64_t d = 0; d < irank; ++d) {
          if (d != axis) {
            strides.push_back(st[static_cast<size_t>(d)]);
          } else {
            for (int64_t e = 0; e < q; ++e) strides.push_back(step[static_cast<size_t>(e)] * st[static_cast<size_t>(axis)]);
          }
        }
        for (int64_t d = 0, k = 0; d < irank; ++d) {  // the output's extents have to be the ones these strides describe
          for (int64_t e = 0; e < (d == axis ? q : 1); ++e, ++k) {
            if (oshape[static_cast<size_t>(k)] != (d == axis ? qshape[static_cast<size_t>(e)] : ishape[static_cast<size_t>(d)])) return std::nullopt;
          }
        }
        offset += base * st[static_cast<size_t>(axis)];
        break;
      }
      case OpKind::Reshape:
      case OpKind::Flatten: {
        ViewTracker tracker(ishape);
        if (!tracker.Reshape(oshape)) return std::nullopt;
        const auto v = tracker.StridesInSource(st);
        if (!v || v->size() != oshape.size()) return std::nullopt;
        strides = *v;
        break;
      }
      default: return std::nullopt;
    }
    if (offset < 0 || offset > INT32_MAX) return std::nullopt;
    return std::make_pair(offset, strides);
  }

  void ElideViews(std::vector<Launch> *fused) {
    // where each step is issued: a fused launch runs at one position for all its members
    std::vector<size_t> issued(steps_.size());
    std::vector<const Launch *> owner(steps_.size(), nullptr);
    for (size_t i = 0; i < steps_.size(); ++i) issued[i] = i;
    for (const Launch &l : *fused) {
      const size_t pos = l.kind == Launch::Kind::MatMulGroup ? l.position : l.members.back();
      for (size_t m : l.members) {
        issued[m] = pos;
        owner[m] = &l;
      }
    }
    // every write of the schedule: (position, bytes, launch it belongs to)
    struct Write {
      size_t position;
      Operand what;
      const Launch *launch;  // null for a single step
      size_t step;           // the single step
    };
    std::vector<Write> writes;
    auto list_writes = [&]() {
      writes.clear();
      for (size_t q = 0; q < steps_.size(); ++q) {
        if (owner[q] == nullptr) writes.push_back({q, steps_[q].out, nullptr, q});
      }
      for (const Launch &l : *fused) {
        const size_t pos = l.kind == Launch::Kind::MatMulGroup ? l.position : l.members.back();
        if (l.group.empty()) writes.push_back({pos, l.out, &l, 0});
        if (l.has_out2) writes.push_back({pos, l.out2, &l, 0});
        for (const Launch &g : l.group) writes.push_back({pos, g.out, &l, 0});
      }
    };
    list_writes();
    std::vector<const Launch *> dissolved;  // copy launches both of whose steps became views
    auto is_dissolved = [&](const Launch *l) { return std::find(dissolved.begin(), dissolved.end(), l) != dissolved.end(); };

    // `seen` = the output of view step(s) starting at position `first`, described inside the source tensor.  Can
    // every reader of `produced` read the source instead?  `skip`: a copy launch that would no longer run.
    auto readers_can_see = [&](size_t first, const Operand &produced, const Operand &seen, const Launch *skip) {
      auto it = readers_.find(produced.name);
      if (it == readers_.end() || it->second.empty()) return false;
      for (size_t r : it->second) {
        if (r <= first) return false;
        const size_t pos = issued[r];
        if (pos < first) return false;  // the reader was hoisted in front of the view step: keep the copy
        for (const Write &w : writes) {
          // nothing may write the source's bytes after the view step and before the reader runs, and the
          // reader's own launch must not write what it now reads through the view
          if (w.launch != nullptr && (w.launch == skip || is_dissolved(w.launch))) continue;
          const bool own = w.launch != nullptr ? w.launch == owner[r] : (owner[r] == nullptr && w.step == r);
          if (w.launch == nullptr && elided_[w.step]) continue;
          if (((w.position > first && w.position < pos) || own) && Alias(w.what, seen)) return false;
        }
        for (size_t q = first + 1; q < pos; ++q) {
          // scratch reserved by a step in between (these kernels do not touch it, but it is not ours to read under)
          const Step &between = steps_[q];
          if (between.has_buffer && seen.space == Operand::Space::Arena && between.buffer_offset < seen.offset + seen.Extent() &&
              seen.offset < between.buffer_offset + between.buffer_bytes) {
            return false;
          }
        }
      }
      return true;
    };
    // step i's output (meta of the step's own output) as the operand its readers would use instead
    auto seen_through = [&](size_t i, const std::pair<int64_t, std::vector<int64_t>> &view) {
      const Step &s = steps_[i];
      Operand seen = s.out;  // keeps the view's meta (shape, type)
      seen.space = s.in0.space;
      seen.name = s.in0.name;
      seen.offset = s.in0.offset;
      seen.viewed = true;
      seen.view_offset = view.first;
      seen.view_strides = view.second;
      seen.source_bytes = s.in0.Extent();
      return seen;
    };
    // rewrite every reader of `produced`: the plan's steps (for later views of this view and for single-step
    // launches) and the operand copies inside fused launches
    auto rewire = [&](const Operand &produced, const Operand &seen) {
      for (size_t r : readers_.at(produced.name)) {
        if (SameTensor(steps_[r].in0, produced)) steps_[r].in0 = seen;
        if (steps_[r].node->IsDoubleInputs() && SameTensor(steps_[r].in1, produced)) steps_[r].in1 = seen;
        rewired_[r] = true;
      }
      for (Launch &l : *fused) {
        for (Operand *op : {&l.a, &l.b, &l.c, &l.d, &l.e}) {
          if (SameTensor(*op, produced) && !op->viewed) *op = seen;
        }
        for (Launch &g : l.group) {
          for (Operand *op : {&g.a, &g.b, &g.c, &g.d, &g.e}) {
            if (SameTensor(*op, produced) && !op->viewed) *op = seen;
          }
        }
      }
    };

    for (size_t i = 0; i < steps_.size(); ++i) {
      if (!steps_[i].node->IsSingleInput()) continue;
      if (taken_[i]) {
        // A Reshape + Transpose (or Transpose + Reshape) pair fused into one strided copy: if the two steps in a
        // row are still one strided view of the source, and the source's bytes last until the readers run, the
        // copy does not have to run either.
        const Launch *l = owner[i];
        if (l == nullptr || is_dissolved(l) || l->members.size() != 2 || l->members[0] != i ||
            (l->kind != Launch::Kind::ReshapeTranspose && l->kind != Launch::Kind::TransposeReshape)) {
          continue;
        }
        const size_t j = l->members[1];
        if (!Elidable(steps_[i].out) || !Elidable(steps_[j].out) || !steps_[j].node->IsSingleInput()) continue;
        const auto first_view = AsView(i);
        if (!first_view) continue;
        const Operand seen_first = seen_through(i, *first_view);
        const Operand saved = steps_[j].in0;
        steps_[j].in0 = seen_first;
        const auto second_view = AsView(j);
        if (!second_view) {
          steps_[j].in0 = saved;
          continue;
        }
        Operand seen = seen_through(j, *second_view);
        seen.source_bytes = seen_first.source_bytes;
        const Operand produced = steps_[j].out;
        if (!readers_can_see(i, produced, seen, l)) {
          // the source's bytes are reused before the last reader runs: with the source in a buffer of its own
          // (if that is all that stands in the way) the readers can look through after all
          Operand apart = seen;
          apart.space = Operand::Space::Private;
          const Operand source = steps_[i].in0;
          steps_[j].in0 = saved;
          const auto root = Underlying(source);
          if (!root || !Movable(*root) || !readers_can_see(i, produced, apart, l)) continue;
          MoveOut(root->name, {fused});
          list_writes();
          --i;  // once more, from the top, with the source where nothing else lives
          continue;
        }
        rewire(produced, seen);
        steps_[i].out = seen_first;
        steps_[j].out = seen;
        elided_[i] = elided_[j] = true;
        dissolved.push_back(l);
        owner[i] = owner[j] = nullptr;
        issued[i] = i;
        issued[j] = j;
        BuildReaders();
        continue;
      }
      if (!Elidable(steps_[i].out)) continue;
      const auto view = AsView(i);
      if (!view) continue;
      const Operand seen = seen_through(i, *view);
      const Operand produced = steps_[i].out;
      if (!readers_can_see(i, produced, seen, nullptr)) {
        Operand apart = seen;
        apart.space = Operand::Space::Private;
        const Operand source = steps_[i].in0;
        // (the source may itself be seen through an elided view: what moves is the tensor underneath)
        const auto root = Underlying(source);
        if (!root || !Movable(*root) || !readers_can_see(i, produced, apart, nullptr)) continue;
        MoveOut(root->name, {fused});
        list_writes();
        --i;
        continue;
      }
      rewire(produced, seen);
      steps_[i].out = seen;
      elided_[i] = true;
      taken_[i] = true;
      BuildReaders();  // names changed: the source gained this step's readers
    }
    fused->erase(std::remove_if(fused->begin(), fused->end(), [&](const Launch &l) { return is_dissolved(&l); }), fused->end());
  }

  // ---- Concat2 inputs written in place ---------------------------------------------------------------------
  // The launch that produces an input of a Concat2 can write it straight into its part of the Concat2's output
  // (every kernel takes output strides), provided nobody else reads the input, and the output's bytes -- which
  // the memory plan reserves only from the Concat2 on -- are touched by nothing else between that launch and the
  // Concat2.  With both inputs in place the Concat2 does not run; with one, it copies the other.  A launch that
  // already writes through folded Reshape / Transpose steps has its strides worked out again for the part.

  // part `side` (0: first input, 1: second) of Concat2 step c's output, as an operand
  Operand ConcatPart(size_t c, int side) const {
    const Step &s = steps_[c];
    const Operand &whole = s.out;
    const auto &shape = whole.meta.GetShape();
    int64_t axis = Attrs(c).axis;
    if (axis < 0) axis += static_cast<int64_t>(shape.size());
    const std::vector<int64_t> strides = LogicalStrides(whole);
    Operand part = whole;
    part.meta = side == 0 ? s.in0.meta : s.in1.meta;
    part.viewed = true;
    part.view_strides = strides;
    part.view_offset = (whole.viewed ? whole.view_offset : 0) +
                       (side == 0 ? 0 : s.in0.meta.GetShape()[static_cast<size_t>(axis)] * strides[static_cast<size_t>(axis)]);
    part.source_bytes = whole.Extent();
    return part;
  }

  // A launch that writes its logical output through folded Reshape / Transpose steps (`view_strides`), asked to
  // write into a tensor of the final shape stored with `final_strides` instead: the strides to use then.
  std::optional<ViewTracker::View> ViewInto(const Launch &l, const std::vector<int64_t> &final_strides) const {
    size_t head = l.members[0];
    int split_dim = -1;
    if (l.kind == Launch::Kind::SoftmaxMatVec) {
      head = l.owner;
      split_dim = 0;  // the kernel takes its batch dim in two parts
    } else if (l.kind == Launch::Kind::Attention) {
      for (size_t m : l.members) {
        if (Kind(m) == OpKind::MatMul) head = m;
      }
    } else if (l.kind != Launch::Kind::MatMulChain) {
      return std::nullopt;
    }
    ViewTracker tracker(steps_[head].out.meta.GetShape());
    for (size_t m : l.members) {
      if (m <= head) continue;
      bool ok = true;
      switch (Kind(m)) {
        case OpKind::Reshape:
        case OpKind::Flatten:
        case OpKind::Squeeze:
        case OpKind::Unsqueeze: ok = tracker.Reshape(steps_[m].out.meta.GetShape()); break;
        case OpKind::Transpose: {
          std::vector<int64_t> perm = Attrs(m).perm;
          if (perm.empty()) {
            for (int64_t d = static_cast<int64_t>(steps_[m].out.meta.GetShape().size()); d-- > 0;) perm.push_back(d);
          }
          ok = tracker.Transpose(perm);
          break;
        }
        default: break;  // elementwise members keep the shape
      }
      if (!ok) return std::nullopt;
    }
    auto v = tracker.Resolve(final_strides, split_dim);
    if (v && l.kind == Launch::Kind::Attention && v->n_inner != 0) return std::nullopt;
    return v;
  }

  // A Concat2 read only by a Reshape / Flatten that keeps the bytes in order (both tensors stored row-major): the
  // Concat2 -- and whoever writes its inputs in place -- can write into the Reshape's buffer, which the memory plan
  // reserves from the Reshape on, and the Reshape does not run.  Nothing else may touch those bytes from the
  // Concat2 to the Reshape, and the Concat2's inputs must not lie under them.
  void WriteIntoReshape(size_t c, const std::vector<size_t> &issued) {
    const Step &cat = steps_[c];
    if (!Elidable(cat.out) || !DefaultLayout(cat.out)) return;
    auto it = readers_.find(cat.out.name);
    if (it == readers_.end() || it->second.size() != 1) return;
    const size_t r = it->second[0];
    if (r <= c || taken_[r] || elided_[r] || (Kind(r) != OpKind::Reshape && Kind(r) != OpKind::Flatten)) return;
    const Step &tail = steps_[r];
    if (!SameTensor(tail.in0, cat.out) || tail.in0.viewed || !Elidable(tail.out) || !DefaultLayout(tail.out) ||
        tail.out.meta.GetType() != cat.out.meta.GetType() || tail.out.meta.GetSize() != cat.out.meta.GetSize()) {
      return;
    }
    Operand whole = tail.out;
    whole.meta = cat.out.meta;
    whole.layout = cat.out.layout;
    whole.viewed = true;
    whole.view_offset = 0;
    whole.view_strides = utils::GenStrides(cat.out.meta.GetShape(), cat.out.layout);
    whole.source_bytes = tail.out.Extent();
    if (Alias(cat.in0, whole) || Alias(cat.in1, whole)) return;
    for (size_t q = 0; q < steps_.size(); ++q) {
      if (q == c || q == r || elided_[q]) continue;
      if (!((q > c && q < r) || (issued[q] >= c && issued[q] <= r))) continue;
      const Step &st = steps_[q];
      if (Alias(st.out, whole) || Alias(st.in0, whole) || (st.node->IsDoubleInputs() && Alias(st.in1, whole))) return;
      if (st.has_buffer && whole.space == Operand::Space::Arena && st.buffer_offset < whole.offset + whole.Extent() &&
          whole.offset < st.buffer_offset + st.buffer_bytes) {
        return;
      }
    }
    steps_[c].out = whole;
    rewired_[c] = true;
    taken_[r] = true;
    filled_[r] = true;
  }

  // ---- Pad inputs written in place ------------------------------------------------------------------------
  // A zero Pad whose input comes from a contraction launch and whose result is only looked at through views (the
  // sliding windows of a span-based convolution: Pad -> Gather -> Transpose [-> Reshape], matched as one copy above):
  // the padded tensor gets a buffer of its own outside the arena -- zero when it is created, and nothing ever writes
  // its border -- the contraction writes its result straight into the interior, the Pad does not run, and the view
  // steps behind it are left to the view elision, whose readers then address the windows inside the padded buffer.
  void PlacePadInputs(std::vector<Launch> *fused) {
    if (std::getenv("FLUIDML_MOVE_OUT_OFF") != nullptr) return;
    for (size_t k = 0; k < fused->size(); ++k) {
      if ((*fused)[k].kind != Launch::Kind::PadViewCopy) continue;
      const Launch copy = (*fused)[k];
      const size_t pad = copy.members[0];
      const Operand x = steps_[pad].in0, padded = steps_[pad].out;
      const bool own_bytes = x.space == Operand::Space::Arena || (x.space == Operand::Space::Private && x.pool.empty());
      if (x.viewed || !own_bytes || !IsFloat(x) || !DefaultLayout(x) || !Elidable(x)) continue;
      if (padded.viewed || !DefaultLayout(padded) || !Elidable(padded) || !Movable(padded)) continue;
      const auto xr = readers_.find(x.name);
      if (xr == readers_.end() || xr->second.size() != 1 || xr->second[0] != pad) continue;
      const auto &pairs = Attrs(pad).pad_pairs;
      const auto &xshape = x.meta.GetShape();
      const auto &pshape = padded.meta.GetShape();
      bool ok = pairs.size() == pshape.size() && xshape.size() == pshape.size();
      for (size_t d = 0; ok && d < pairs.size(); ++d) {
        ok = std::get<0>(pairs[d]) >= 0 && std::get<1>(pairs[d]) >= 0 &&
             xshape[d] + std::get<0>(pairs[d]) + std::get<1>(pairs[d]) == pshape[d];
      }
      if (!ok) continue;
      // the launch (or member of a group) that writes x, as a plain MatMul chain: it takes any output strides
      const auto made = producer_.find(x.name);
      if (made == producer_.end()) continue;
      Launch *member = nullptr;
      size_t position = 0;
      for (Launch &l : *fused) {
        const size_t pos = l.kind == Launch::Kind::MatMulGroup ? l.position : l.members.back();
        if (l.group.empty()) {
          if (SameTensor(l.out, x) && !l.out.viewed && l.members.back() == made->second) member = &l, position = pos;
        } else {
          for (Launch &g : l.group) {
            if (SameTensor(g.out, x) && !g.out.viewed && g.members.back() == made->second) member = &g, position = pos;
          }
        }
      }
      if (member == nullptr || member->kind != Launch::Kind::MatMulChain || !member->view_strides.empty() ||
          member->has_skip || member->has_out2 || member->norm_mode != 0 ||
          !member->norm_stats_out.empty() || position >= pad) {
        continue;
      }
      MoveOut(padded.name, {fused});
      const Operand whole = steps_[pad].out;  // (where it lives now)
      const std::vector<int64_t> strides = LogicalStrides(whole);
      Operand interior = whole;
      interior.meta = x.meta;
      interior.viewed = true;
      interior.view_strides = strides;
      interior.view_offset = 0;
      for (size_t d = 0; d < pairs.size(); ++d) interior.view_offset += std::get<0>(pairs[d]) * strides[d];
      interior.source_bytes = whole.Extent();
      for (Launch &l : *fused) {
        // (a group carries a copy of one member's output operand as its own)
        if (!l.group.empty() && SameTensor(l.out, x) && !l.out.viewed) l.out = interior;
      }
      member->out = interior;
      steps_[made->second].out = interior;
      filled_[pad] = true;  // nothing runs at the Pad's place
      for (size_t m = 1; m < copy.members.size(); ++m) taken_[copy.members[m]] = false;
      fused->erase(fused->begin() + static_cast<std::ptrdiff_t>(k));
      --k;
      BuildReaders();
    }
  }

  void PlaceConcatInputs(std::vector<Launch> *fused) {
    std::vector<size_t> issued(steps_.size());
    std::vector<Launch *> owner(steps_.size(), nullptr);
    for (size_t i = 0; i < steps_.size(); ++i) issued[i] = i;
    for (Launch &l : *fused) {
      const size_t pos = l.kind == Launch::Kind::MatMulGroup ? l.position : l.members.back();
      for (size_t m : l.members) {
        issued[m] = pos;
        owner[m] = &l;
      }
    }
    MarkSilent(*fused);
    auto really_read = [&](const Operand &op) {
      if (op.viewed) return true;
      auto it = producer_.find(op.name);
      return it == producer_.end() || !silent_[it->second];
    };
    for (size_t c = 0; c < steps_.size(); ++c) {
      if (taken_[c] || Kind(c) != OpKind::Concat2) continue;
      const Step &cat = steps_[c];
      const auto &oshape = cat.out.meta.GetShape();
      int64_t axis = Attrs(c).axis;
      if (axis < 0) axis += static_cast<int64_t>(oshape.size());
      if (axis < 0 || axis >= static_cast<int64_t>(oshape.size()) || cat.out.viewed || SameTensor(cat.in0, cat.in1)) continue;
      if (cat.in0.meta.GetShape().size() != oshape.size() || cat.in1.meta.GetShape().size() != oshape.size()) continue;
      WriteIntoReshape(c, issued);
      for (int side = 0; side < 2; ++side) {
        const Operand &x = side == 0 ? cat.in0 : cat.in1;
        if (x.viewed || !Elidable(x) || x.meta.GetType() != cat.out.meta.GetType()) continue;
        auto it = readers_.find(x.name);
        if (it == readers_.end() || it->second.size() != 1 || it->second[0] != c) continue;
        // the step that writes x, and the launch it runs in
        std::optional<size_t> producer;
        for (size_t q = 0; q < c; ++q) {
          if (!elided_[q] && SameTensor(steps_[q].out, x) && !steps_[q].out.viewed) producer = q;
        }
        if (!producer) continue;
        Launch *l = owner[*producer];
        if (l != nullptr) {
          // (a launch with a residual addend or a per-channel gate reads those through the strides of its own output
          // tensor -- the kernels take no separate strides for them -- so it cannot write into a part of a wider one)
          const bool plain_out = l->group.empty() && SameTensor(l->out, x) && !l->out.viewed && !l->has_out2 &&
                                 !l->has_skip && !l->has_gate;
          const bool kind_ok = l->kind == Launch::Kind::MatMulChain || l->kind == Launch::Kind::GemmChain ||
                               l->kind == Launch::Kind::ConvChain || l->kind == Launch::Kind::ElementwiseChain ||
                               l->kind == Launch::Kind::DivAddSoftmax || l->kind == Launch::Kind::AddLayerNorm ||
                               l->kind == Launch::Kind::Attention || l->kind == Launch::Kind::MulAdd ||
                               l->kind == Launch::Kind::AddAdd ||
                               (l->kind == Launch::Kind::SoftmaxMatVec && !l->view_strides.empty());
          if (!plain_out || !kind_ok) continue;
        } else if (taken_[*producer] || placed_[*producer] != 0) {
          continue;
        }
        const size_t from = issued[*producer];
        if (from >= c) continue;
        Operand target = ConcatPart(c, side);
        // a launch that writes through folded views: its logical output's strides inside the part
        std::optional<ViewTracker::View> into;
        if (l != nullptr && !l->view_strides.empty()) {
          into = ViewInto(*l, target.view_strides);
          if (!into || l->has_skip) continue;
        }
        auto clear_for = [&](const Operand &target) {
          bool ok = true;
          for (size_t q = 0; q < steps_.size() && ok; ++q) {
            if (q == c || elided_[q]) continue;
            if (l != nullptr ? owner[q] == l : q == *producer) continue;
            const bool in_range = (q >= from && q <= c) || (issued[q] >= from && issued[q] <= c);
            if (!in_range) continue;
            const Step &st = steps_[q];
            // the other input's producer may already write its own part of the same output
            const bool other_part = st.out.viewed && SameTensor(st.out, cat.out) && placed_[c] != 0;
            // (intermediates of a fused launch are neither written nor read)
            if (!other_part && !silent_[q] && Alias(st.out, target)) ok = false;
            if ((really_read(st.in0) && Alias(st.in0, target)) ||
                (st.node->IsDoubleInputs() && really_read(st.in1) && Alias(st.in1, target))) ok = false;
            if (st.has_buffer && target.space == Operand::Space::Arena && st.buffer_offset < target.offset + target.Extent() &&
                target.offset < st.buffer_offset + st.buffer_bytes) {
              ok = false;
            }
          }
          // the producer's own inputs must not lie under the bytes it now writes
          for (size_t m : (l != nullptr ? l->members : std::vector<size_t>{*producer})) {
            const Step &st = steps_[m];
            if ((really_read(st.in0) && Alias(st.in0, target)) ||
                (st.node->IsDoubleInputs() && really_read(st.in1) && Alias(st.in1, target))) {
              ok = false;
            }
          }
          if (l != nullptr) {
            for (const Operand *op : {&l->a, &l->b, &l->c, &l->d, &l->e}) {
              if (!op->name.empty() && Alias(*op, target)) ok = false;
            }
          }
          return ok;
        };
        // nothing else may touch the output's bytes from the producer's launch up to the Concat2; where the plan has
        // other tenants there, the Concat2's output gets a buffer of its own outside the arena (a part already
        // written in place moves with it: its checks held for the planned bytes and hold for bytes nobody shares)
        if (!clear_for(target)) {
          Operand apart = target;
          apart.space = Operand::Space::Private;
          apart.offset = 0;
          apart.pool.clear();
          if (!Movable(cat.out) || !clear_for(apart)) continue;
          MoveOut(cat.out.name, {fused});
          target = ConcatPart(c, side);
        }
        steps_[*producer].out = target;
        if (l != nullptr) l->out = target;
        else rewired_[*producer] = true;
        if (into) {
          l->view_strides = into->strides;
          l->n_inner = into->n_inner;
          l->stride_outer = into->stride_outer;
        }
        placed_[c] |= side == 0 ? 1 : 2;
      }
      if (placed_[c] != 0) taken_[c] = true;
    }
    silent_.clear();
  }

  OpKind Kind(size_t i) const { return steps_[i].node->GetKind(); }
  const flow::Attrs &Attrs(size_t i) const { return steps_[i].node->GetAttrs(); }

  // the only reader of step i's output, if it has exactly one, is free, comes later and the tensor is elidable
  std::optional<size_t> SoleReader(size_t i) const {
    const Operand &o = steps_[i].out;
    if (!Elidable(o)) return std::nullopt;
    auto it = readers_.find(o.name);
    if (it == readers_.end() || it->second.size() != 1) return std::nullopt;
    const size_t j = it->second[0];
    if (j <= i || taken_[j]) return std::nullopt;
    return j;
  }

  // For a double-input step `j` reading `produced`: the other operand (nullopt if both are `produced`).
  std::optional<Operand> Other(size_t j, const Operand &produced) const {
    const Step &s = steps_[j];
    if (!s.node->IsDoubleInputs()) return std::nullopt;
    const bool l = SameTensor(s.in0, produced), r = SameTensor(s.in1, produced);
    if (l == r) return std::nullopt;
    return l ? s.in1 : s.in0;
  }

  // Issuing member m's reads at position `last` is safe when no foreign step in between writes over them.
  bool Safe(const std::vector<size_t> &members, const std::vector<std::pair<size_t, Operand>> &external) const {
    const size_t last = members.back();
    for (const auto &[m, op] : external) {
      for (size_t s = m + 1; s < last; ++s) {
        if (std::find(members.begin(), members.end(), s) != members.end()) continue;
        if (!moved_.empty() && moved_[s] != SIZE_MAX && moved_[s] <= m) continue;  // runs before the first read now
        if (elided_[s] || (!silent_.empty() && silent_[s])) continue;  // never written
        if (Alias(steps_[s].out, op)) return false;
      }
      // steps a group moved into the window from outside it
      for (size_t s = 0; s < moved_.size(); ++s) {
        if (moved_[s] == SIZE_MAX || (s > m && s < last)) continue;
        if (moved_[s] > m && moved_[s] < last && Alias(steps_[s].out, op)) return false;
      }
    }
    // the chain's own output must not overwrite an external input another member still needs: the fused kernel
    // reads and writes concurrently, the unfused sequence only tolerates that element for element
    return true;
  }

  // Safe, or made safe by giving the operands whose bytes get other tenants in the window a buffer of their own
  // outside the arena (`moves`: their names, to be moved once the caller has decided for the launch).
  bool SafeWithMoves(const std::vector<size_t> &members, const std::vector<std::pair<size_t, Operand>> &external,
                     std::vector<std::string> *moves) const {
    std::vector<std::string> wanted;
    for (const auto &e : external) {
      if (Safe(members, {e})) continue;
      const auto root = Underlying(e.second);
      if (!root || !Movable(*root)) return false;
      wanted.push_back(root->name);
    }
    moves->insert(moves->end(), wanted.begin(), wanted.end());
    return true;
  }

  static double Bytes(std::initializer_list<const Operand *> ops) {
    double n = 0;
    std::vector<const Operand *> seen;
    for (const Operand *o : ops) {
      bool dup = false;
      for (const Operand *p : seen) dup = dup || SameTensor(*o, *p);
      if (!dup) n += static_cast<double>(o->meta.GetSize());
      seen.push_back(o);
    }
    return n;
  }

  double Flops(const std::vector<size_t> &members) const {
    double f = 0;
    for (size_t m : members) f += steps_[m].flops;
    return f;
  }

  // a fused kernel reads its inputs while it writes its output: the output may only overlap an input exactly
  // (same tensor, element-for-element in-place), never partially
  bool OutputDisjoint(const Operand &out, std::initializer_list<const Operand *> ins) const {
    for (const Operand *in : ins) {
      if (Alias(out, *in)) return false;
    }
    return true;
  }

  // fl_ew_op of a unary step with at most one scalar constant, -1 if the step is not one
  int UnaryOp(size_t i) const {
    if (!IsFloat(steps_[i].out) || !IsFloat(steps_[i].in0)) return -1;
    switch (Kind(i)) {
      case OpKind::AddConstant: return FL_EW_ADD_C;
      case OpKind::SubConstantLhs: return FL_EW_RSUB_C;
      case OpKind::MulConstant: return FL_EW_MUL_C;
      case OpKind::DivConstantRhs: return FL_EW_DIV_C;
      case OpKind::Pow: return FL_EW_POW_C;
      case OpKind::Erf: return FL_EW_ERF;
      case OpKind::Relu: return FL_EW_RELU;
      case OpKind::Tanh: return FL_EW_TANH;
      case OpKind::Sqrt: return FL_EW_SQRT;
      case OpKind::Neg: return FL_EW_NEG;
      default: return -1;
    }
  }

  // fl_ew_op of a binary step that combines the running value `value` with the chain input `root`, -1 otherwise
  int BinaryWithRoot(size_t j, const Operand &value, const Operand &root) const {
    const Step &s = steps_[j];
    if (!s.node->IsDoubleInputs() || !IsFloat(s.out)) return -1;
    const bool value_left = SameTensor(s.in0, value) && SameTensor(s.in1, root);
    const bool value_right = SameTensor(s.in1, value) && SameTensor(s.in0, root);
    if (value_left == value_right) return -1;
    switch (Kind(j)) {
      case OpKind::AddCommon: return FL_EW_ADD_X;
      case OpKind::MulCommon: return FL_EW_MUL_X;
      case OpKind::SubCommon: return value_left ? FL_EW_SUB_X : FL_EW_RSUB_X;
      case OpKind::DivCommon: return value_left ? FL_EW_DIV_X : FL_EW_RDIV_X;
      default: return -1;
    }
  }

  struct Chain {
    std::vector<size_t> members;
    fl_ew_program program{};
  };

  // The longest chain of free elementwise steps that starts at `first` (a unary step reading `root`) and
  // whose intermediate values each have one reader.  Binary steps may combine the value with `root` again.
  Chain Follow(const Operand &root, size_t first) const {
    Chain c;
    size_t cur = first;
    c.members.push_back(first);
    c.program.op[0] = UnaryOp(first);
    c.program.c[0] = static_cast<float>(Attrs(first).value);
    c.program.n = 1;
    while (c.program.n < FL_EW_MAX_STEPS) {
      const auto j = SoleReader(cur);
      if (!j || steps_[*j].out.meta.GetShape() != root.meta.GetShape()) break;
      int op = -1;
      float value = 0.0f;
      if (steps_[*j].node->IsSingleInput()) {
        op = UnaryOp(*j);
        value = static_cast<float>(Attrs(*j).value);
      } else {
        op = BinaryWithRoot(*j, steps_[cur].out, root);
      }
      if (op < 0) break;
      c.program.op[c.program.n] = op;
      c.program.c[c.program.n] = value;
      ++c.program.n;
      c.members.push_back(*j);
      cur = *j;
    }
    return c;
  }

  // The chain that consumes `root` completely (every reader of `root` is a member), so `root` need not be written.
  std::optional<Chain> ConsumingChain(size_t producer) const {
    const Operand &root = steps_[producer].out;
    if (!Elidable(root) || !IsFloat(root)) return std::nullopt;
    auto it = readers_.find(root.name);
    if (it == readers_.end()) return std::nullopt;
    std::optional<size_t> first;
    for (size_t r : it->second) {
      if (r <= producer || taken_[r]) return std::nullopt;
      if (steps_[r].node->IsSingleInput() && UnaryOp(r) >= 0 && SameTensor(steps_[r].in0, root) &&
          steps_[r].out.meta.GetShape() == root.meta.GetShape()) {
        if (first) return std::nullopt;  // two unary readers: two chains, keep the tensor
        first = r;
      }
    }
    if (!first) return std::nullopt;
    Chain c = Follow(root, *first);
    for (size_t r : it->second) {
      if (std::find(c.members.begin(), c.members.end(), r) == c.members.end()) return std::nullopt;
    }
    return c;
  }

  std::optional<Launch> MatchContraction(size_t i) {
    const Step &head = steps_[i];
    if (!IsFloat(head.out)) return std::nullopt;
    Launch l;
    l.a = head.in0;
    l.b = head.in1;
    l.owner = i;
    l.members = {i};
    size_t value_step = i;  // the step whose output the elementwise chain starts from
    if (Kind(i) == OpKind::MatMul) {
      l.kind = Launch::Kind::MatMulChain;
      // MatMul -> AddCommon(rank-1 constant bias over the last dim)
      if (const auto j = SoleReader(i); j && Kind(*j) == OpKind::AddCommon) {
        const auto bias = Other(*j, head.out);
        const auto &shape = head.out.meta.GetShape();
        if (bias && bias->space == Operand::Space::Constant && IsFloat(*bias) && bias->meta.GetShape().size() == 1 &&
            bias->meta.GetShape()[0] == shape.back() && steps_[*j].out.meta.GetShape() == shape) {
          l.c = *bias;
          l.has_c = true;
          l.members.push_back(*j);
          value_step = *j;
        }
      }
    } else if (Kind(i) == OpKind::GemmConstantWeightsBias) {
      l.kind = Launch::Kind::GemmChain;
    } else {
      l.kind = Launch::Kind::ConvChain;
    }
    const size_t without_chain = l.members.size();
    if (const auto chain = ConsumingChain(value_step)) {
      l.members.insert(l.members.end(), chain->members.begin(), chain->members.end());
      l.chain = chain->program;
    }
    if (l.kind == Launch::Kind::MatMulChain) {
      if (auto wider = WithAddends(i, l)) return wider;
    }
    // MatMul only: trailing Reshape / Transpose steps that merely re-address the result are folded into the
    // kernel's output strides (the head split and merge copies of an attention block)
    if (l.kind == Launch::Kind::MatMulChain) {
      // the longest run of view steps whose target buffer is safe to write from here; a shorter run leaves the
      // rest to the view elision (a Reshape of what the kernel wrote is then read in place)
      for (size_t limit = SIZE_MAX; limit > 0;) {
        Launch with_views = l;
        const size_t taken = AppendViews(i, &with_views, limit);
        if (taken == 0) break;
        if (with_views.members.size() >= 2 && Safe(with_views.members, {{i, l.a}, {i, l.b}}) &&
            OutputDisjoint(with_views.out, {&l.a, &l.b})) {
          with_views.bytes = l.has_c ? Bytes({&l.a, &l.b, &l.c, &with_views.out}) : Bytes({&l.a, &l.b, &with_views.out});
          with_views.flops = Flops(with_views.members);
          return with_views;
        }
        limit = taken - 1;
      }
    }
    if (l.kind == Launch::Kind::ConvChain) {
      if (auto wider = WithGateAndSkip(i, l)) return wider;
      if (auto wider = WithMean(i, l)) return wider;
    }
    // longest variant whose late reads are safe: with the chain, then without it
    for (int attempt = 0; attempt < 2; ++attempt) {
      if (l.members.size() < 2) return std::nullopt;  // nothing fused
      l.out = steps_[l.members.back()].out;
      // (a result the plan put over bytes of an operand -- dead by then in the serial order, still read by this
      // launch -- moves to a buffer of its own once the sweep is over)
      const bool disjoint = OutputDisjoint(l.out, {&l.a, &l.b});
      std::vector<std::string> moves;
      if ((disjoint || Movable(l.out)) && SafeWithMoves(l.members, {{i, l.a}, {i, l.b}}, &moves)) {
        if (!disjoint) moves.push_back(l.out.name);
        pending_moves_.insert(pending_moves_.end(), moves.begin(), moves.end());
        l.bytes = l.has_c ? Bytes({&l.a, &l.b, &l.c, &l.out}) : Bytes({&l.a, &l.b, &l.out});
        l.bytes += static_cast<double>(steps_[i].kernel->GetConstantBytes());
        l.flops = Flops(l.members);
        return l;
      }
      l.members.resize(without_chain);
      l.chain = fl_ew_program{};
    }
    return std::nullopt;
  }

  // A MatMul chain (already matched in `plain`) whose value goes through one or two AddCommon with tensors of its
  // own shape and layout (a residual connection; GPT-NeoX's x + attention + mlp): the tensors become operands of
  // the launch, added in the epilogue in the order of the steps.  The kernel's instantiations with extra operands
  // want the right operand stored n-fastest.
  std::optional<Launch> WithAddends(size_t i, const Launch &plain) {
    if (const char *v = std::getenv("FLUIDML_MATMUL_ADDENDS"); v != nullptr && std::string(v) == "0") return std::nullopt;
    const Step &head = steps_[i];
    if (!IsFloat(head.in1) || head.in1.viewed || !DefaultLayout(head.in1) || head.in1.meta.GetShape().size() < 2) return std::nullopt;
    std::vector<size_t> adds;
    std::vector<Operand> tensors;
    size_t value = plain.members.back();
    while (adds.size() < 2) {
      const auto j = SoleReader(value);
      if (!j || Kind(*j) != OpKind::AddCommon) break;
      const Operand &v = steps_[value].out;
      const auto other = Other(*j, v);
      if (!other || !IsFloat(*other) || other->viewed || other->space == Operand::Space::Constant ||
          other->meta.GetShape() != v.meta.GetShape() || steps_[*j].out.meta.GetShape() != v.meta.GetShape()) {
        break;
      }
      adds.push_back(*j);
      tensors.push_back(*other);
      value = *j;
    }
    for (size_t n = adds.size(); n >= 1; --n) {
      Launch l = plain;
      std::vector<std::pair<size_t, Operand>> external = {{i, l.a}, {i, l.b}};
      bool ok = true;
      for (size_t k = 0; k < n; ++k) {
        l.members.push_back(adds[k]);
        external.push_back({adds[k], tensors[k]});
      }
      l.out = steps_[l.members.back()].out;
      bool clash = !OutputDisjoint(l.out, {&l.a, &l.b});
      for (size_t k = 0; k < n; ++k) {
        ok = ok && tensors[k].layout == l.out.layout;
        clash = clash || Alias(l.out, tensors[k]);
      }
      std::vector<std::string> moves;
      if (!ok || (clash && !Movable(l.out)) || !SafeWithMoves(l.members, external, &moves)) continue;
      // (the plan put the sum over bytes of an operand the launch still reads: the sum moves out of the arena)
      if (clash) moves.push_back(l.out.name);
      pending_moves_.insert(pending_moves_.end(), moves.begin(), moves.end());
      l.d = tensors[0];
      l.has_skip = true;
      if (n == 2) {
        l.e = tensors[1];
        l.has_skip2 = true;
      }
      l.bytes = l.has_c ? Bytes({&l.a, &l.b, &l.c, &l.out}) : Bytes({&l.a, &l.b, &l.out});
      for (size_t k = 0; k < n; ++k) l.bytes += static_cast<double>(tensors[k].meta.GetSize());
      l.flops = Flops(l.members);
      return l;
    }
    return std::nullopt;
  }

  // A depthwise 2-d convolution (with the chain already matched in `plain`) one of whose readers is the ReduceMean
  // over both spatial dims (the squeeze of a squeeze-and-excitation block): the kernel that owns a whole channel
  // plane per workgroup delivers the mean with the result.  The launch runs at the ReduceMean's position and writes
  // both tensors, so every other reader of the result has to come after it.
  std::optional<Launch> WithMean(size_t i, const Launch &plain) {
    const Step &conv = steps_[i];
    const auto &in_shape = conv.in0.meta.GetShape();
    const auto &w_shape = conv.in1.meta.GetShape();
    if (in_shape.size() != 4 || w_shape.size() != 4 || Attrs(i).group == 1 || Attrs(i).group != in_shape[1] || w_shape[1] != 1) return std::nullopt;
    const size_t value = plain.members.back();
    const Operand &result = steps_[value].out;
    if (!Elidable(result) || !IsFloat(result)) return std::nullopt;
    auto it = readers_.find(result.name);
    if (it == readers_.end()) return std::nullopt;
    std::optional<size_t> mean;
    for (size_t r : it->second) {
      if (Kind(r) != OpKind::ReduceMean || taken_[r] || r <= value) continue;
      const flow::Attrs &at = Attrs(r);
      std::vector<int64_t> axes(at.axes);
      for (int64_t &ax : axes) ax = ax < 0 ? ax + 4 : ax;
      std::sort(axes.begin(), axes.end());
      if (at.keepdims && axes == std::vector<int64_t>{2, 3} && (!mean || r < *mean)) mean = r;
    }
    if (!mean) return std::nullopt;
    for (size_t r : it->second) {
      if (r != *mean && std::find(plain.members.begin(), plain.members.end(), r) == plain.members.end() && r < *mean) return std::nullopt;
    }
    Launch l = plain;
    l.members.push_back(*mean);
    l.out = result;
    l.out2 = steps_[*mean].out;
    l.has_out2 = true;
    if (!IsFloat(l.out2) || !Elidable(l.out2)) return std::nullopt;
    // (the plan may put the result over the convolution's input, dead by then in the plan but read by this launch,
    // which runs at the ReduceMean's place: the result then moves out of the arena)
    const bool clash = !OutputDisjoint(l.out, {&l.a, &l.b});
    if (!Safe(l.members, {{i, l.a}, {i, l.b}}) || (clash && !Movable(l.out)) || !OutputDisjoint(l.out2, {&l.a, &l.b, &l.out})) return std::nullopt;
    if (clash) pending_moves_.push_back(l.out.name);
    l.bytes = Bytes({&l.a, &l.b, &l.out}) + static_cast<double>(steps_[i].kernel->GetConstantBytes()) + static_cast<double>(l.out2.meta.GetSize());
    l.flops = Flops(l.members);
    return l;
  }

  static bool DefaultLayout(const Operand &o) {
    if (o.viewed) return false;
    for (size_t d = 0; d < o.layout.size(); ++d) {
      if (o.layout[d] != d) return false;
    }
    return true;
  }

  // A convolution `i` (with the chain already matched in `plain`) whose input is a MulCommon of a tensor with one
  // factor per channel (the gate of a squeeze-and-excitation block) and / or whose result goes into an AddCommon
  // with a tensor of its own shape (a skip connection): both become operands of the launch.  Only where the launch
  // is a plain contraction (1x1, unit stride, no padding, default layouts): that kernel scales the rows of its
  // right operand while staging them (one image) and adds a tensor with the output's strides in its epilogue.
  std::optional<Launch> WithGateAndSkip(size_t i, const Launch &plain) {
    const Step &conv = steps_[i];
    const flow::Attrs &at = Attrs(i);
    const auto &in_shape = conv.in0.meta.GetShape();
    bool pointwise = at.group == 1 && in_shape.size() <= 4 && IsFloat(conv.in0) && DefaultLayout(conv.in1) &&
                     DefaultLayout(conv.out) && (conv.in0.viewed ? false : DefaultLayout(conv.in0));
    const auto &w_shape = conv.in1.meta.GetShape();
    for (size_t d = 2; d < w_shape.size() && pointwise; ++d) pointwise = w_shape[d] == 1;
    for (size_t d = 0; d < at.strides.size() && pointwise; ++d) pointwise = at.strides[d] == 1;
    if (Kind(i) == OpKind::ConvWithPadding) {
      for (size_t d = 0; d < at.pads.size() && pointwise; ++d) pointwise = at.pads[d] == 0;
    }
    if (!pointwise) return std::nullopt;
    // the gate
    std::optional<size_t> mul;
    Operand x, gate;
    if (auto it = producer_.find(conv.in0.name); it != producer_.end() && in_shape[0] == 1) {
      const size_t m = it->second;
      bool gated = Kind(m) == OpKind::MulCommon && !taken_[m] && m < i;
      if (gated) {
        const auto reader = SoleReader(m);
        gated = reader && *reader == i;
      }
      if (gated) {
        const Step &ms = steps_[m];
        for (int side = 0; side < 2 && !mul; ++side) {
          const Operand &full = side == 0 ? ms.in0 : ms.in1, &factor = side == 0 ? ms.in1 : ms.in0;
          const auto &fs = factor.meta.GetShape();
          bool ok = IsFloat(full) && IsFloat(factor) && full.meta.GetShape() == in_shape && fs.size() == in_shape.size() &&
                    fs[1] == in_shape[1] && DefaultLayout(full) && !SameTensor(full, factor);
          for (size_t d = 0; d < fs.size() && ok; ++d) ok = d == 1 || fs[d] == 1;
          if (ok) {
            mul = m;
            x = full;
            gate = factor;
          }
        }
      }
    }
    // the skip connection
    std::optional<size_t> add;
    Operand skip;
    if (const auto j = SoleReader(plain.members.back()); j && Kind(*j) == OpKind::AddCommon) {
      const Operand &value = steps_[plain.members.back()].out;
      const auto other = Other(*j, value);
      if (other && IsFloat(*other) && !other->viewed && other->meta.GetShape() == value.meta.GetShape() &&
          steps_[*j].out.meta.GetShape() == value.meta.GetShape() && other->layout == steps_[*j].out.layout &&
          other->space != Operand::Space::Constant) {
        add = *j;
        skip = *other;
      }
    }
    // ... or a MulCommon with a tensor of the result's shape behind it, directly or behind a Transpose that swaps the
    // channel and pixel dims of a 1-d convolution (ConvBERT's span-based kernel: the convolved keys times the
    // queries): the launch multiplies in its epilogue and writes the product, through transposed strides where
    // the Transpose stood
    bool factor = false, transposed = false;
    std::optional<size_t> between;  // the Transpose
    if (!add) {
      size_t value = plain.members.back();
      std::optional<size_t> j = SoleReader(value);
      if (j && Kind(*j) == OpKind::Transpose && in_shape.size() == 3 && Attrs(*j).perm == std::vector<int64_t>{0, 2, 1} &&
          DefaultLayout(steps_[*j].out) && IsFloat(steps_[*j].out)) {
        between = *j;
        value = *j;
        j = SoleReader(value);
      }
      if (j && Kind(*j) == OpKind::MulCommon) {
        const Operand &v = steps_[value].out;
        const auto other = Other(*j, v);
        if (other && IsFloat(*other) && !other->viewed && DefaultLayout(*other) && other->meta.GetShape() == v.meta.GetShape() &&
            steps_[*j].out.meta.GetShape() == v.meta.GetShape() && DefaultLayout(steps_[*j].out) && IsFloat(steps_[*j].out) &&
            other->space != Operand::Space::Constant) {
          add = *j;
          skip = *other;
          factor = true;
          transposed = between.has_value();
        }
      }
    }
    // `op` (default layout, the shape behind the Transpose) addressed with the dims of the convolution's own result
    auto swapped = [&](const Operand &op) {
      Operand seen = op;
      seen.meta = conv.out.meta;
      const std::vector<int64_t> st = LogicalStrides(op);
      seen.viewed = true;
      seen.view_offset = 0;
      seen.view_strides = {st[0], st[2], st[1]};
      seen.source_bytes = op.Extent();
      return seen;
    };
    // the widest variant whose late reads are safe
    for (int variant = 0; variant < 3; ++variant) {
      const bool with_gate = variant != 2, with_skip = variant != 1;
      if ((with_gate && !mul) || (with_skip && !add) || (!with_gate && !with_skip)) continue;
      Launch l = plain;
      std::vector<std::pair<size_t, Operand>> external = {{i, l.b}};
      if (with_gate) {
        l.members.insert(l.members.begin(), *mul);
        l.a = x;
        l.c = gate;
        l.has_gate = true;
        external.push_back({*mul, x});
        external.push_back({*mul, gate});
      } else {
        external.push_back({i, l.a});
      }
      if (with_skip) {
        if (between) l.members.push_back(*between);
        l.members.push_back(*add);
        l.d = transposed ? swapped(skip) : skip;
        l.has_skip = true;
        l.skip_is_factor = factor;
        external.push_back({*add, skip});
      }
      l.out = steps_[l.members.back()].out;
      const Operand planned_out = l.out;
      if (with_skip && transposed) l.out = swapped(l.out);
      std::vector<std::string> moves;
      const bool clash = !OutputDisjoint(l.out, {&l.a, &l.b}) || (with_gate && Alias(l.out, l.c)) || (with_skip && Alias(l.out, l.d));
      // the plan reuses bytes of an operand for the result (dead by then in the serial order, still read by this
      // launch): the result moves to a buffer of its own once the sweep is over; so does an operand whose bytes get
      // another tenant before the launch, which now reads it later than planned, has run
      if ((clash && !Movable(planned_out)) || !SafeWithMoves(l.members, external, &moves)) continue;
      if (clash) moves.push_back(planned_out.name);
      pending_moves_.insert(pending_moves_.end(), moves.begin(), moves.end());
      l.bytes = Bytes({&l.a, &l.b, &l.out}) + static_cast<double>(steps_[i].kernel->GetConstantBytes());
      if (with_gate) l.bytes += static_cast<double>(l.c.meta.GetSize());
      if (with_skip) l.bytes += static_cast<double>(l.d.meta.GetSize());
      l.flops = Flops(l.members);
      return l;
    }
    return std::nullopt;
  }

  // Softmax over the K <= 16 logits of [B, K, 1] whose only reader multiplies [B, M, K] with it (and whatever
  // Reshape / Transpose views MatchContraction folds behind that MatMul): one launch of fluidml_hip_softmax_matvec
  std::optional<Launch> MatchSoftmaxMatVec(size_t i) {
    const Step &soft = steps_[i];
    const auto &vs = soft.in0.meta.GetShape();
    if (!IsFloat(soft.in0) || !IsFloat(soft.out) || vs.size() != 3 || vs[2] != 1 || vs[1] > 16) return std::nullopt;
    const int64_t axis = Attrs(i).axis < 0 ? Attrs(i).axis + 3 : Attrs(i).axis;
    if (axis != 1) return std::nullopt;
    const auto j = SoleReader(i);
    if (!j || Kind(*j) != OpKind::MatMul || !SameTensor(steps_[*j].in1, soft.out) || SameTensor(steps_[*j].in0, soft.out)) {
      return std::nullopt;
    }
    const auto &as = steps_[*j].in0.meta.GetShape();
    if (!IsFloat(steps_[*j].in0) || as.size() != 3 || as[0] != vs[0] || as[2] != vs[1]) return std::nullopt;
    Launch l;
    if (auto chain = MatchContraction(*j); chain && chain->kind == Launch::Kind::MatMulChain && !chain->has_c &&
                                           chain->chain.n == 0 && chain->n_inner == 0) {
      l = *chain;  // MatMul + the views folded behind it
    } else {
      l.members = {*j};
      l.a = steps_[*j].in0;
      l.out = steps_[*j].out;
    }
    l.kind = Launch::Kind::SoftmaxMatVec;
    l.owner = *j;
    l.b = soft.in0;
    l.members.insert(l.members.begin(), i);
    // (operands or a result the plan has other tenants for in the launch's window move out of the arena)
    std::vector<std::string> moves;
    const bool clash = !OutputDisjoint(l.out, {&l.a, &l.b});
    if (clash && !Movable(l.out)) return std::nullopt;
    if (!SafeWithMoves(l.members, {{i, l.b}, {*j, l.a}}, &moves)) return std::nullopt;
    if (clash) moves.push_back(l.out.name);
    pending_moves_.insert(pending_moves_.end(), moves.begin(), moves.end());
    l.bytes = Bytes({&l.a, &l.b, &l.out});
    l.flops = Flops(l.members);
    return l;
  }

  // A convolution that is a matrix-vector product per image: group 1, one input pixel, one tap, no padding
  // (the two convolutions of a squeeze-and-excitation block behind the global pooling).
  bool PointwiseOnOnePixel(size_t i) const {
    if (Kind(i) != OpKind::ConvWithoutPadding) return false;
    const Step &st = steps_[i];
    const auto &in = st.in0.meta.GetShape(), &w = st.in1.meta.GetShape(), &out = st.out.meta.GetShape();
    if (!IsFloat(st.in0) || !IsFloat(st.in1) || !IsFloat(st.out) || Attrs(i).group != 1) return false;
    if (in.size() < 3 || w.size() != in.size() || out.size() != in.size() || w[1] != in[1]) return false;
    for (size_t d = 2; d < in.size(); ++d) {
      if (in[d] != 1 || w[d] != 1 || out[d] != 1) return false;
    }
    return true;
  }

  // Conv -> chain -> Conv -> chain on one-pixel tensors: one launch of fluidml_hip_pointwise_conv_pair
  std::optional<Launch> MatchConvPair(size_t i) {
    if (!PointwiseOnOnePixel(i)) return std::nullopt;
    Launch l;
    l.kind = Launch::Kind::ConvPair;
    l.a = steps_[i].in0;
    l.b = steps_[i].in1;
    l.owner = i;
    l.members = {i};
    size_t last = i;
    if (const auto chain = ConsumingChain(i)) {
      l.members.insert(l.members.end(), chain->members.begin(), chain->members.end());
      l.chain = chain->program;
      last = chain->members.back();
    }
    const auto j = SoleReader(last);
    if (!j || !PointwiseOnOnePixel(*j) || !SameTensor(steps_[*j].in0, steps_[last].out)) return std::nullopt;
    // the kernel's limits, so that the launch can never be refused at replay time
    if (steps_[i].in0.meta.GetShape()[1] > 4096 || steps_[*j].in0.meta.GetShape()[1] > 512 ||
        steps_[i].in0.meta.GetShape()[0] > 65535) {
      return std::nullopt;
    }
    l.members.push_back(*j);
    l.c = steps_[*j].in1;
    l.owner2 = *j;
    if (const auto chain = ConsumingChain(*j)) {
      l.members.insert(l.members.end(), chain->members.begin(), chain->members.end());
      l.chain2 = chain->program;
    }
    std::sort(l.members.begin(), l.members.end());
    l.out = steps_[l.members.back()].out;
    if (!Safe(l.members, {{i, l.a}, {i, l.b}, {*j, l.c}}) || !OutputDisjoint(l.out, {&l.a, &l.b, &l.c})) return std::nullopt;
    l.bytes = Bytes({&l.a, &l.b, &l.c, &l.out}) + static_cast<double>(steps_[i].kernel->GetConstantBytes()) +
              static_cast<double>(steps_[*j].kernel->GetConstantBytes());
    l.flops = Flops(l.members);
    return l;
  }

  // Extends `l` (a MatMulChain headed by step `head`) by the longest run of single-reader Reshape / Transpose
  // steps after which the contraction's logical output is still a strided view of the final tensor.
  // At most `limit` view steps are taken; returns how many were (0: none).
  size_t AppendViews(size_t head, Launch *l, size_t limit = SIZE_MAX) const {
    ViewTracker tracker(steps_[head].out.meta.GetShape());
    size_t cur = l->members.back();
    std::vector<size_t> views;
    size_t best = 0;
    ViewTracker::View best_view;
    while (views.size() < limit) {
      const auto j = SoleReader(cur);
      if (!j || !IsFloat(steps_[*j].out)) break;
      bool ok = false;
      switch (Kind(*j)) {
        case OpKind::Reshape:
        case OpKind::Flatten:
        case OpKind::Squeeze:
        case OpKind::Unsqueeze: ok = tracker.Reshape(steps_[*j].out.meta.GetShape()); break;
        case OpKind::Transpose: {
          std::vector<int64_t> perm = Attrs(*j).perm;
          if (perm.empty()) {
            for (int64_t d = static_cast<int64_t>(steps_[*j].out.meta.GetShape().size()); d-- > 0;) perm.push_back(d);
          }
          ok = tracker.Transpose(perm);
          break;
        }
        default: break;
      }
      if (!ok) break;
      views.push_back(*j);
      cur = *j;
      const Operand &o = steps_[*j].out;
      if (auto v = tracker.Resolve(utils::GenStrides(o.meta.GetShape(), o.layout))) {
        best = views.size();
        best_view = *v;
      }
    }
    if (best == 0) return 0;
    l->members.insert(l->members.end(), views.begin(), views.begin() + static_cast<std::ptrdiff_t>(best));
    l->out = steps_[l->members.back()].out;
    l->view_strides = best_view.strides;
    l->n_inner = best_view.n_inner;
    l->stride_outer = best_view.stride_outer;
    return best;
  }

  // Two Rotary launches with the same tables and extents, the second of which follows the first with nothing of
  // consequence in between (the queries and the keys of a layer), become one launch at the position of the second:
  // the first one's reads move there (nothing in between may write what it reads), its output appears later than
  // planned (nothing in between may read it), and neither may write what the other reads.
  void PairRotary(std::vector<Launch> *fused) const {
    if (const char *v = std::getenv("FLUIDML_ROTARY_PAIR"); v != nullptr && std::string(v) == "0") return;
    std::vector<bool> used(fused->size(), false);
    std::vector<Launch> result;
    for (size_t i = 0; i < fused->size(); ++i) {
      if (used[i]) continue;
      const Launch &x = (*fused)[i];
      size_t partner = fused->size();
      if (x.kind == Launch::Kind::Rotary) {
        for (size_t j = 0; j < fused->size() && partner == fused->size(); ++j) {
          const Launch &y = (*fused)[j];
          if (j == i || used[j] || y.kind != Launch::Kind::Rotary || y.members.back() <= x.members.back()) continue;
          if (!SameTensor(x.b, y.b) || !SameTensor(x.c, y.c) || x.b.viewed || y.b.viewed || x.c.viewed || y.c.viewed ||
              x.axis != y.axis || x.a.meta.GetShape() != y.a.meta.GetShape()) {
            continue;
          }
          std::vector<size_t> members = x.members;
          members.insert(members.end(), y.members.begin(), y.members.end());
          std::sort(members.begin(), members.end());
          if (!Safe(members, {{x.members.front(), x.a}, {x.members.front(), x.b}, {x.members.front(), x.c},
                              {y.members.front(), y.a}})) {
            continue;
          }
          bool ok = !Alias(x.out, y.out) && !Alias(x.out, y.a) && !Alias(y.out, x.a);
          // nobody reads the first result before the common position
          auto rd = readers_.find(x.out.name);
          if (rd != readers_.end()) {
            for (size_t r : rd->second) ok = ok && r > y.members.back();
          }
          // its bytes, planned from its last member on, stay its own until then (written later than planned)
          for (size_t s = x.members.back() + 1; s < y.members.back() && ok; ++s) {
            if (std::find(members.begin(), members.end(), s) != members.end() || elided_[s]) continue;
            const Step &st = steps_[s];
            if (Alias(st.out, x.out) || Alias(st.in0, x.out) || (st.node->IsDoubleInputs() && Alias(st.in1, x.out))) ok = false;
          }
          if (ok) partner = j;
        }
      }
      if (partner == fused->size()) {
        result.push_back(x);
        used[i] = true;
        continue;
      }
      const Launch &y = (*fused)[partner];
      Launch g;
      g.kind = Launch::Kind::RotaryPair;
      g.members = x.members;
      g.members.insert(g.members.end(), y.members.begin(), y.members.end());
      std::sort(g.members.begin(), g.members.end());
      g.group = {x, y};
      g.position = g.members.back();
      g.a = x.a;
      g.b = x.b;
      g.c = x.c;
      g.axis = x.axis;
      g.out = y.out;
      g.bytes = x.bytes + y.bytes;
      g.flops = x.flops + y.flops;
      used[i] = used[partner] = true;
      result.push_back(std::move(g));
    }
    *fused = std::move(result);
  }

  // MatMulChains that read the same left operand with the same extents (the query / key / value projections)
  // become one launch at the position of the last of them, provided that moving the earlier ones there
  // crosses no reader of their outputs and no write to what they read.
  void GroupSiblings(std::vector<Launch> *fused) {
    auto compatible = [&](const Launch &x, const Launch &y) {
      if (x.kind != Launch::Kind::MatMulChain || y.kind != Launch::Kind::MatMulChain || x.has_skip || y.has_skip) return false;
      const Step &hx = steps_[x.members[0]], &hy = steps_[y.members[0]];
      const auto &shape = hx.out.meta.GetShape();
      int64_t batch = 1;
      for (size_t d = 0; d + 2 < shape.size(); ++d) batch *= shape[d];
      return SameTensor(x.a, y.a) && x.a.layout == y.a.layout && batch == 1 && shape == hy.out.meta.GetShape() &&
             x.b.space == Operand::Space::Constant && y.b.space == Operand::Space::Constant &&
             x.b.meta.GetShape() == y.b.meta.GetShape() && x.b.layout == y.b.layout && x.has_c == y.has_c &&
             InnerCompatible(x, y, shape.back()) && x.chain.n == y.chain.n &&
             std::equal(x.chain.op, x.chain.op + x.chain.n, y.chain.op) &&
             std::equal(x.chain.c, x.chain.c + x.chain.n, y.chain.c);
    };
    std::vector<bool> used(fused->size(), false);
    std::vector<Launch> result;
    for (size_t i = 0; i < fused->size(); ++i) {
      if (used[i]) continue;
      std::vector<size_t> set = {i};
      int64_t inner = (*fused)[i].n_inner;  // the one non-zero column split of the set, if any
      for (size_t j = i + 1; j < fused->size() && set.size() < 4; ++j) {
        const Launch &y = (*fused)[j];
        if (used[j] || !compatible((*fused)[i], y)) continue;
        if (y.n_inner != 0 && inner != 0 && y.n_inner != inner) continue;
        if (y.n_inner != 0) inner = y.n_inner;
        set.push_back(j);
      }
      // the largest prefix of the candidates that can meet at the position of one of them
      size_t position = 0;
      std::vector<std::string> moves;  // outputs of hoisted members that need a buffer outside the arena
      while (set.size() >= 2) {
        bool found = false;
        for (size_t k : set) {
          moves.clear();
          if (CanGroupAt(*fused, set, (*fused)[k].members.back(), &moves)) {
            position = (*fused)[k].members.back();
            found = true;
            break;
          }
        }
        if (found) break;
        set.pop_back();
      }
      if (set.size() >= 2) {
        for (const std::string &name : moves) MoveOut(name, {fused, &result});
      }
      if (set.size() < 2) {
        result.push_back((*fused)[i]);
        used[i] = true;
        continue;
      }
      Launch g;
      g.kind = Launch::Kind::MatMulGroup;
      for (size_t k : set) {
        used[k] = true;
        const Launch &m = (*fused)[k];
        g.members.insert(g.members.end(), m.members.begin(), m.members.end());
        g.flops += m.flops;
        g.bytes += m.bytes - (k == set[0] ? 0.0 : static_cast<double>(m.a.meta.GetSize()));
        g.group.push_back(m);
        // a member whose columns are one strided run joins members with split columns by splitting its run
        Launch &added = g.group.back();
        if (added.n_inner == 0 && inner != 0) {
          added.n_inner = inner;
          added.stride_outer = inner * (added.view_strides.empty() ? LogicalStrides(added.out).back() : added.view_strides.back());
        }
      }
      std::sort(g.members.begin(), g.members.end());
      std::sort(g.group.begin(), g.group.end(), [](const Launch &x, const Launch &y) { return x.members.back() < y.members.back(); });
      g.a = g.group[0].a;
      g.out = g.group.back().out;
      g.position = position;
      result.push_back(std::move(g));
    }
    *fused = std::move(result);
  }

  // Two chains can share a launch if their column addressing can be made the same: equal splits of the last
  // output dim, or one of them unsplit (its columns are then one strided run, which any split describes too).
  static bool InnerCompatible(const Launch &x, const Launch &y, int64_t columns) {
    if (x.n_inner == y.n_inner) return true;
    if (x.n_inner != 0 && y.n_inner != 0) return false;
    const int64_t inner = x.n_inner != 0 ? x.n_inner : y.n_inner;
    return columns % inner == 0;  // (a member without folded views writes its own output: one run per row as well)
  }

  // Can every launch of `set` be issued at step position `position` (the last member of one of them)?
  // `moves` collects the outputs of hoisted members whose planned bytes are in use at the earlier position: the
  // caller moves those tensors out of the arena.
  bool CanGroupAt(const std::vector<Launch> &fused, const std::vector<size_t> &set, size_t position,
                  std::vector<std::string> *moves) const {
    auto moved = [&](const Operand &op) { return std::find(moves->begin(), moves->end(), op.name) != moves->end(); };

    std::vector<size_t> members;
    for (size_t k : set) members.insert(members.end(), fused[k].members.begin(), fused[k].members.end());
    auto is_member = [&](size_t s) { return std::find(members.begin(), members.end(), s) != members.end(); };
    for (size_t k : set) {
      const Launch &l = fused[k];
      const size_t own = l.members.back();
      if (own <= position) {
        // delayed: its reads of the left operand (weights and bias are constants) move from the chain's head
        // to `position`, and its output appears later than planned
        for (size_t s = l.members[0] + 1; s < position; ++s) {
          if (!is_member(s) && Alias(steps_[s].out, l.a)) return false;
        }
        auto it = readers_.find(l.out.name);
        if (it != readers_.end()) {
          for (size_t r : it->second) {
            if (r <= position) return false;
          }
        }
      } else {
        // hoisted: the left operand must exist already, and the output's bytes, reserved only from `own` on,
        // must not be touched by anything that runs between the new and the planned position
        if (l.members[0] <= position) return false;  // part of the chain already ran: not a pure hoist
        auto producer_before = [&](const Operand &op) {
          if (op.space == Operand::Space::Constant || op.space == Operand::Space::Interface) {
            // constants always exist; interface tensors are graph inputs unless a step writes them
            for (size_t s = position; s < steps_.size(); ++s) {
              if (SameTensor(steps_[s].out, op)) return false;
            }
            return true;
          }
          for (size_t s = 0; s < position; ++s) {
            if (SameTensor(steps_[s].out, op)) return true;
          }
          return false;
        };
        if (!producer_before(l.a)) return false;
        // (a step inside a fused launch that is not its last never writes its output, and what it reads from
        // such a step is never read)
        auto exists = [&](const Operand &op) {
          if (silent_.empty() || op.viewed) return true;
          const auto it = producer_.find(op.name);
          return it == producer_.end() || !silent_[it->second];
        };
        bool in_use = false;
        for (size_t s = position; s <= own && !in_use; ++s) {
          if (is_member(s)) continue;
          const Step &st = steps_[s];
          const bool unwritten = !silent_.empty() && silent_[s];
          if (!unwritten && Alias(st.out, l.out)) in_use = true;
          if (exists(st.in0) && Alias(st.in0, l.out)) in_use = true;
          if (st.node->IsDoubleInputs() && exists(st.in1) && Alias(st.in1, l.out)) in_use = true;
          if (st.has_buffer && !unwritten && l.out.space == Operand::Space::Arena && st.buffer_offset < l.out.offset + l.out.meta.GetSize() &&
              l.out.offset < st.buffer_offset + st.buffer_bytes) {
            in_use = true;  // scratch of a step in between (untouched by these kernels, but reserved)
          }
        }
        if (in_use) {
          if (!Movable(l.out)) return false;
          moves->push_back(l.out.name);
        }
      }
      // the output must not overlap what a member reads at the common position
      for (size_t other : set) {
        if (Alias(l.out, fused[other].a) && !moved(l.out)) {
          if (own <= position || !Movable(l.out)) return false;
          moves->push_back(l.out.name);
        }
      }
    }
    // outputs of different members are live together from the later one's planned position on, but a hoisted
    // output and a not-yet-dead neighbour could still collide: all outputs pairwise disjoint
    for (size_t x : set) {
      for (size_t y : set) {
        if (x < y && Alias(fused[x].out, fused[y].out) && !moved(fused[x].out) && !moved(fused[y].out)) return false;
      }
    }
    return true;
  }

  // Two or more elementwise steps on a tensor that stays live (or is a graph input).
  std::optional<Launch> MatchElementwise(size_t i) {
    const Step &head = steps_[i];
    if (head.in0.meta.GetShape() != head.out.meta.GetShape()) return std::nullopt;
    Chain c = Follow(head.in0, i);
    if (c.members.size() < 2) return std::nullopt;
    Launch l;
    l.kind = Launch::Kind::ElementwiseChain;
    l.members = c.members;
    l.chain = c.program;
    l.a = head.in0;
    l.out = steps_[l.members.back()].out;
    if (!Safe(l.members, {{i, l.a}})) return std::nullopt;
    // in place is fine element for element (same bytes, same layout); any other overlap is not
    if (Alias(l.out, l.a) && !(l.out.space == Operand::Space::Arena && l.a.space == Operand::Space::Arena &&
                               l.out.offset == l.a.offset && l.out.layout == l.a.layout)) {
      return std::nullopt;
    }
    l.bytes = Bytes({&l.a, &l.out});
    return l;
  }

  // MulCommon whose only reader is an AddCommon: a * b + c in one launch
  std::optional<Launch> MatchMulAdd(size_t i) {
    const Step &mul = steps_[i];
    if (!IsFloat(mul.out) || !IsFloat(mul.in0) || !IsFloat(mul.in1)) return std::nullopt;
    const auto j = SoleReader(i);
    if (!j || Kind(*j) != OpKind::AddCommon || !IsFloat(steps_[*j].out)) return std::nullopt;
    const auto other = Other(*j, mul.out);
    if (!other || !IsFloat(*other)) return std::nullopt;
    Launch l;
    l.kind = Launch::Kind::MulAdd;
    l.members = {i, *j};
    l.a = mul.in0;
    l.b = mul.in1;
    l.c = *other;
    l.out = steps_[*j].out;
    if (!Safe(l.members, {{i, l.a}, {i, l.b}, {*j, l.c}}) || !OutputDisjoint(l.out, {&l.a, &l.b, &l.c})) return std::nullopt;
    l.bytes = Bytes({&l.a, &l.b, &l.c, &l.out});
    return l;
  }

  // ---- rotary position embedding ---------------------------------------------------------------------------
  // The free step that produces `o` when `reader` is the only step reading it.
  std::optional<size_t> ProducerFor(const Operand &o, size_t reader) const {
    if (o.viewed) return std::nullopt;
    const auto it = producer_.find(o.name);
    if (it == producer_.end() || taken_[it->second] || it->second >= reader) return std::nullopt;
    const auto only = SoleReader(it->second);
    if (!only || *only != reader) return std::nullopt;
    return it->second;
  }

  // Slice step i as the range [begin, begin + length) of the last axis with everything else whole.
  std::optional<std::pair<int64_t, int64_t>> LastAxisRange(size_t i) const {
    if (Kind(i) != OpKind::Slice) return std::nullopt;
    const auto &ishape = steps_[i].in0.meta.GetShape();
    const auto &oshape = steps_[i].out.meta.GetShape();
    if (ishape.size() != oshape.size() || ishape.empty()) return std::nullopt;
    const int64_t rank = static_cast<int64_t>(ishape.size());
    for (int64_t d = 0; d + 1 < rank; ++d) {
      if (ishape[static_cast<size_t>(d)] != oshape[static_cast<size_t>(d)]) return std::nullopt;
    }
    const flow::Attrs &at = Attrs(i);
    if (at.starts.size() != at.axes.size() || at.steps.size() != at.axes.size()) return std::nullopt;
    int64_t begin = 0;
    for (size_t n = 0; n < at.axes.size(); ++n) {
      const int64_t ax = at.axes[n] < 0 ? at.axes[n] + rank : at.axes[n];
      if (ax < 0 || ax >= rank || at.steps[n] != 1) return std::nullopt;
      int64_t b = at.starts[n];
      if (b < 0) b += ishape[static_cast<size_t>(ax)];
      if (ax == rank - 1) begin = b;
      else if (b != 0) return std::nullopt;
    }
    if (begin < 0 || begin + oshape.back() > ishape.back()) return std::nullopt;
    return std::make_pair(begin, oshape.back());
  }

  bool LastAxis(size_t concat) const {
    const int64_t rank = static_cast<int64_t>(steps_[concat].out.meta.GetShape().size());
    const int64_t axis = Attrs(concat).axis;
    return (axis < 0 ? axis + rank : axis) == rank - 1;
  }

  // x_rot * cos + concat(-x_rot[.., h:], x_rot[.., :h]) * sin, matched from its AddCommon (step i); when x_rot is
  // itself the slice x[.., :R] and the sum is concatenated with x[.., R:], those steps join too, and so does a
  // Transpose of the result (written through permuted strides).  One launch of fluidml_hip_rotary.
  std::optional<Launch> MatchRotary(size_t i) {
    // FLUIDML_ROTARY=0 leaves the steps to the general mechanisms (views, Concat2 inputs written in place)
    if (const char *v = std::getenv("FLUIDML_ROTARY"); v != nullptr && std::string(v) == "0") return std::nullopt;
    const Step &add = steps_[i];
    if (!IsFloat(add.out) || SameTensor(add.in0, add.in1)) return std::nullopt;
    const auto p0 = ProducerFor(add.in0, i), p1 = ProducerFor(add.in1, i);
    if (!p0 || !p1 || Kind(*p0) != OpKind::MulCommon || Kind(*p1) != OpKind::MulCommon) return std::nullopt;
    for (int swap = 0; swap < 2; ++swap) {
      const size_t m1 = swap ? *p1 : *p0, m2 = swap ? *p0 : *p1;  // m1: x_rot * cos, m2: turned * sin
      for (int side = 0; side < 2; ++side) {
        const Operand &turned = side ? steps_[m2].in1 : steps_[m2].in0;
        const Operand &sin_t = side ? steps_[m2].in0 : steps_[m2].in1;
        const auto c1 = ProducerFor(turned, m2);
        if (!c1 || Kind(*c1) != OpKind::Concat2 || !LastAxis(*c1)) continue;
        const auto neg = ProducerFor(steps_[*c1].in0, *c1), s1 = ProducerFor(steps_[*c1].in1, *c1);
        if (!neg || !s1 || Kind(*neg) != OpKind::Neg) continue;
        const auto s2 = ProducerFor(steps_[*neg].in0, *neg);
        if (!s2) continue;
        const auto r1 = LastAxisRange(*s1), r2 = LastAxisRange(*s2);
        if (!r1 || !r2 || !SameTensor(steps_[*s1].in0, steps_[*s2].in0)) continue;
        const Operand x_rot = steps_[*s1].in0;
        const int64_t rot = x_rot.meta.GetShape().back(), half = rot / 2;
        if (rot % 2 != 0 || r1->first != 0 || r1->second != half || r2->first != half || r2->second != half) continue;
        const bool left = SameTensor(steps_[m1].in0, x_rot), right = SameTensor(steps_[m1].in1, x_rot);
        if (left == right) continue;
        const Operand &cos_t = left ? steps_[m1].in1 : steps_[m1].in0;
        if (add.out.meta.GetShape() != x_rot.meta.GetShape() || !IsFloat(x_rot) || !IsFloat(cos_t) || !IsFloat(sin_t)) continue;
        // the tables: rot values along the last axis, leading dims broadcast to x_rot's
        bool tables = true;
        for (const Operand *t : {&cos_t, &sin_t}) {
          const auto &ts = t->meta.GetShape();
          const auto &xs = x_rot.meta.GetShape();
          tables = tables && !ts.empty() && ts.size() <= xs.size() && ts.back() == rot;
          for (size_t d = 0; tables && d + 1 < ts.size(); ++d) {
            const int64_t want = xs[xs.size() - ts.size() + d];
            tables = ts[d] == 1 || ts[d] == want;
          }
        }
        if (!tables) continue;
        Launch l;
        l.kind = Launch::Kind::Rotary;
        l.members = {m1, *s1, *s2, *neg, *c1, m2, i};
        l.a = x_rot;
        l.b = cos_t;
        l.c = sin_t;
        l.axis = rot;
        l.out = add.out;
        size_t first_x = std::min({m1, *s1, *s2});
        // the outer Slice / Concat2 pair around a partial rotation
        Launch whole = l;
        bool widened = false;
        if (const auto c2 = SoleReader(i); c2 && Kind(*c2) == OpKind::Concat2 && LastAxis(*c2) &&
                                           SameTensor(steps_[*c2].in0, add.out) && !x_rot.viewed) {
          const auto sp = ProducerFor(steps_[*c2].in1, *c2);
          const auto pr = producer_.find(x_rot.name);
          if (sp && pr != producer_.end() && !taken_[pr->second] && Elidable(x_rot)) {
            const size_t sr = pr->second;
            const auto rr = LastAxisRange(sr), rp = LastAxisRange(*sp);
            const auto rd = readers_.find(x_rot.name);
            std::vector<size_t> expect = {m1, *s1, *s2};
            std::sort(expect.begin(), expect.end());
            std::vector<size_t> have = rd != readers_.end() ? rd->second : std::vector<size_t>{};
            std::sort(have.begin(), have.end());
            if (rr && rp && have == expect && SameTensor(steps_[sr].in0, steps_[*sp].in0) && rr->first == 0 &&
                rr->second == rot && rp->first == rot && rp->first + rp->second == steps_[sr].in0.meta.GetShape().back()) {
              whole.members.push_back(sr);
              whole.members.push_back(*sp);
              whole.members.push_back(*c2);
              whole.a = steps_[sr].in0;
              whole.out = steps_[*c2].out;
              first_x = std::min(sr, *sp);
              widened = true;
            }
          }
        }
        Launch &best = widened ? whole : l;
        std::sort(best.members.begin(), best.members.end());
        // a Transpose of the result: written through permuted strides
        Launch turned_out = best;
        bool transposed = false;
        if (const auto t = SoleReader(best.members.back()); t && Kind(*t) == OpKind::Transpose &&
                                                          Attrs(*t).perm.size() == best.out.meta.GetShape().size()) {
          turned_out.members.push_back(*t);
          turned_out.perm = Attrs(*t).perm;
          turned_out.out = steps_[*t].out;
          transposed = true;
        }
        auto finish = [&](Launch *x, size_t x_from) {
          // (operands or a result the plan has other tenants for in the launch's window move out of the arena)
          std::vector<std::string> moves;
          const bool clash = !OutputDisjoint(x->out, {&x->a, &x->b, &x->c});
          if (clash && !Movable(x->out)) return false;
          if (!SafeWithMoves(x->members, {{x_from, x->a}, {m1, x->b}, {m2, x->c}}, &moves)) return false;
          if (clash) moves.push_back(x->out.name);
          pending_moves_.insert(pending_moves_.end(), moves.begin(), moves.end());
          x->bytes = Bytes({&x->a, &x->b, &x->c, &x->out});
          x->flops = 0;
          return true;
        };
        if (transposed && finish(&turned_out, widened ? first_x : std::min({m1, *s1, *s2}))) return turned_out;
        if (finish(&best, widened ? first_x : std::min({m1, *s1, *s2}))) return best;
        if (widened) {
          std::sort(l.members.begin(), l.members.end());
          if (finish(&l, std::min({m1, *s1, *s2}))) return l;
        }
        return std::nullopt;
      }
    }
    return std::nullopt;
  }

  // GatherAdd (one addend) -> AddLayerNorm over the last dim, the embedding block of a BERT-style encoder: one launch
  // (fluidml_hip_gather_add_layer_normalization).  Where the GatherAdd's addend is itself a looked-up embedding with no
  // other reader, that lookup joins too.  Every operand in its default layout; sums in the order of the steps.
  void FuseEmbeddings(std::vector<Launch> *fused) {
    if (const char *v = std::getenv("FLUIDML_EMBEDDING"); v != nullptr && std::string(v) == "0") return;
    auto only_reader = [&](const Operand &o, size_t reader) {
      if (!Elidable(o)) return false;
      const auto it = readers_.find(o.name);
      return it != readers_.end() && it->second.size() == 1 && it->second[0] == reader;
    };
    // `t` has the trailing dims of `out` with nothing but ones in front (it repeats along out's leading dims)
    auto repeats = [](const std::vector<int64_t> &t, const std::vector<int64_t> &out) {
      if (t.empty() || t.size() > out.size() || t.back() != out.back()) return false;
      bool ones = false;
      for (size_t i = 1; i <= out.size(); ++i) {
        const int64_t have = i <= t.size() ? t[t.size() - i] : 1;
        if (!ones && have == out[out.size() - i]) continue;
        if (have != 1) return false;
        ones = true;
      }
      return true;
    };
    for (size_t n = 0; n < fused->size(); ++n) {
      const Launch norm = (*fused)[n];
      if (norm.kind != Launch::Kind::AddLayerNorm || norm.norm_mode != 0 || !norm.norm_stats_out.empty()) continue;
      const std::vector<int64_t> &shape = norm.out.meta.GetShape();
      const int64_t rank = static_cast<int64_t>(shape.size());
      if (rank < 2 || (norm.axis != rank - 1 && norm.axis != -1) || shape.back() > FL_GATHER_LAYER_NORM_MAX_LEN) continue;
      size_t g = fused->size();
      for (size_t k = 0; k < fused->size() && g == fused->size(); ++k) {
        const Launch &cand = (*fused)[k];
        if (cand.kind != Launch::Kind::GatherAdd || cand.has_c) continue;
        if (!SameTensor(cand.out, norm.a) && !SameTensor(cand.out, norm.b)) continue;
        if (only_reader(cand.out, norm.members.front())) g = k;
      }
      if (g == fused->size()) continue;
      const Launch gather = (*fused)[g];
      const Operand &third = SameTensor(gather.out, norm.a) ? norm.b : norm.a;
      if (SameTensor(third, gather.out) || !IsFloat(third) || !DefaultLayout(third) || !DefaultLayout(norm.out) ||
          !DefaultLayout(gather.a) || !DefaultLayout(gather.b) || gather.out.meta.GetShape() != shape ||
          !repeats(third.meta.GetShape(), shape) || !repeats(gather.b.meta.GetShape(), shape)) {
        continue;
      }
      // a table of rows: the result has one dim more than the indices
      if (steps_[gather.owner].kernel->GetConstant(0) == nullptr ||
          static_cast<int64_t>(gather.a.meta.GetShape().size()) != rank - 1) {
        continue;
      }
      Launch l;
      l.kind = Launch::Kind::GatherAddLayerNorm;
      l.members = gather.members;
      l.members.insert(l.members.end(), norm.members.begin(), norm.members.end());
      l.a = gather.a;
      l.b = gather.b;
      l.c = third;
      l.has_c = true;
      l.out = norm.out;
      l.owner = gather.owner;
      l.norm_owner = norm.owner;
      l.s0 = norm.s0;
      std::vector<std::pair<size_t, Operand>> external = {{gather.members.front(), l.a}, {norm.members.front(), l.c}};
      // the addend of the lookup: a second lookup that nobody else reads
      size_t second = SIZE_MAX;
      if (const auto p = producer_.find(gather.b.name); p != producer_.end() && !taken_[p->second] &&
                                                        Kind(p->second) == OpKind::GatherConstantDataTensor) {
        const Step &st = steps_[p->second];
        if (IsFloat(st.out) && st.kernel->GetConstant(0) != nullptr && only_reader(st.out, gather.members[1]) &&
            st.out.meta.GetShape() == shape && DefaultLayout(st.in0) &&
            st.in0.meta.GetShape() == gather.a.meta.GetShape()) {
          second = p->second;
        }
      }
      Launch with_second = l;
      if (second != SIZE_MAX) {
        with_second.members.push_back(second);
        std::sort(with_second.members.begin(), with_second.members.end());
        with_second.b = steps_[second].in0;
        with_second.has_gate = true;
        with_second.owner2 = second;
        auto ext = external;
        ext.push_back({second, with_second.b});
        if (Safe(with_second.members, ext) && OutputDisjoint(with_second.out, {&with_second.a, &with_second.b, &with_second.c})) {
          l = with_second;
        } else {
          second = SIZE_MAX;
        }
      }
      if (second == SIZE_MAX) {
        std::sort(l.members.begin(), l.members.end());
        external.push_back({gather.members[1], l.b});
        if (!Safe(l.members, external) || !OutputDisjoint(l.out, {&l.a, &l.b, &l.c})) continue;
      }
      l.bytes = Bytes({&l.a, &l.c, &l.out}) + 2.0 * static_cast<double>(l.out.meta.GetSize()) +
                static_cast<double>(steps_[norm.owner].kernel->GetConstantBytes());
      if (second != SIZE_MAX) taken_[second] = true;
      (*fused)[n] = std::move(l);
      fused->erase(fused->begin() + static_cast<std::ptrdiff_t>(g));
      if (g < n) --n;
    }
  }

  // GatherConstantDataTensor -> AddCommon [-> AddCommon] (an embedding lookup and the embeddings added to it)
  std::optional<Launch> MatchGatherAdd(size_t i) {
    const Step &gather = steps_[i];
    if (!IsFloat(gather.out) || steps_[i].kernel->GetConstant(0) == nullptr) return std::nullopt;
    const auto j = SoleReader(i);
    if (!j || Kind(*j) != OpKind::AddCommon || !IsFloat(steps_[*j].out)) return std::nullopt;
    if (steps_[*j].out.meta.GetShape() != gather.out.meta.GetShape()) return std::nullopt;
    const auto first = Other(*j, gather.out);
    if (!first || !IsFloat(*first)) return std::nullopt;
    Launch l;
    l.kind = Launch::Kind::GatherAdd;
    l.members = {i, *j};
    l.a = gather.in0;
    l.b = *first;
    l.out = steps_[*j].out;
    l.owner = i;
    std::vector<std::pair<size_t, Operand>> external = {{i, l.a}, {*j, l.b}};
    Launch longer = l;
    if (const auto k = SoleReader(*j); k && Kind(*k) == OpKind::AddCommon && IsFloat(steps_[*k].out) &&
                                       steps_[*k].out.meta.GetShape() == gather.out.meta.GetShape()) {
      if (const auto second = Other(*k, steps_[*j].out); second && IsFloat(*second)) {
        longer.members.push_back(*k);
        longer.c = *second;
        longer.has_c = true;
        longer.out = steps_[*k].out;
        auto ext = external;
        ext.push_back({*k, longer.c});
        if (Safe(longer.members, ext) && OutputDisjoint(longer.out, {&longer.a, &longer.b, &longer.c})) {
          longer.bytes = Bytes({&longer.a, &longer.b, &longer.c, &longer.out}) + static_cast<double>(longer.out.meta.GetSize());
          return longer;
        }
      }
    }
    if (!Safe(l.members, external) || !OutputDisjoint(l.out, {&l.a, &l.b})) return std::nullopt;
    l.bytes = Bytes({&l.a, &l.b, &l.out}) + static_cast<double>(l.out.meta.GetSize());  // + the gathered rows
    return l;
  }

  // AddCommon -> AddCommon (two residuals): (a + b) + c in one launch, rounded like the two kernels
  std::optional<Launch> MatchAddAdd(size_t i) {
    const Step &first = steps_[i];
    if (!IsFloat(first.out) || !IsFloat(first.in0) || !IsFloat(first.in1)) return std::nullopt;
    const auto j = SoleReader(i);
    if (!j || Kind(*j) != OpKind::AddCommon || !IsFloat(steps_[*j].out)) return std::nullopt;
    const auto other = Other(*j, first.out);
    if (!other || !IsFloat(*other)) return std::nullopt;
    Launch l;
    l.kind = Launch::Kind::AddAdd;
    l.members = {i, *j};
    l.a = first.in0;
    l.b = first.in1;
    l.c = *other;
    l.out = steps_[*j].out;
    if (!Safe(l.members, {{i, l.a}, {i, l.b}, {*j, l.c}}) || !OutputDisjoint(l.out, {&l.a, &l.b, &l.c})) return std::nullopt;
    l.bytes = Bytes({&l.a, &l.b, &l.c, &l.out});
    return l;
  }

  std::optional<Launch> MatchSoftmax(size_t i) {
    const Step &div = steps_[i];
    if (!IsFloat(div.out)) return std::nullopt;
    const auto j = SoleReader(i);
    if (!j || Kind(*j) != OpKind::AddCommon) return std::nullopt;
    const auto mask = Other(*j, div.out);
    if (!mask || !IsFloat(*mask)) return std::nullopt;
    const Step &add = steps_[*j];
    if (add.out.meta.GetShape() != div.out.meta.GetShape()) return std::nullopt;
    const auto k = SoleReader(*j);
    if (!k || Kind(*k) != OpKind::Softmax) return std::nullopt;
    Launch l;
    l.kind = Launch::Kind::DivAddSoftmax;
    l.members = {i, *j, *k};
    l.a = div.in0;
    l.b = *mask;
    l.out = steps_[*k].out;
    l.s0 = Attrs(i).value;
    l.axis = steps_[*k].node->GetAxis();
    if (!Safe(l.members, {{i, l.a}, {*j, l.b}})) return std::nullopt;
    // a row is read completely before it is written: in-place on the input is fine, partial overlap is not
    if (Alias(l.out, l.a) && !(l.out.space == Operand::Space::Arena && l.out.offset == l.a.offset && l.out.layout == l.a.layout)) return std::nullopt;
    if (Alias(l.out, l.b)) return std::nullopt;
    l.bytes = Bytes({&l.a, &l.b, &l.out});
    return l;
  }

  // silent_[s]: step s sits inside a fused launch and is not the member whose output the launch writes
  void MarkSilent(const std::vector<Launch> &fused) {
    silent_.assign(steps_.size(), false);
    for (const Launch &l : fused) {
      for (size_t m : l.members) silent_[m] = true;
      if (l.group.empty()) silent_[l.members.back()] = false;
      if (l.has_out2 && l.members.size() >= 2) silent_[l.members[l.members.size() - 2]] = false;
      for (const Launch &g : l.group) silent_[g.members.back()] = false;
    }
  }

  // A Softmax over a few logits left alone in front of the matrix-vector product that reads it (the
  // product possibly with views folded behind it): refused in the first sweep where a view step in between, elided
  // since, had its output planned over the logits.
  void RetrySoftmaxMatVec(std::vector<Launch> *fused) {
    moved_.assign(steps_.size(), SIZE_MAX);
    MarkSilent(*fused);
    for (const Launch &l : *fused) {
      if (l.kind != Launch::Kind::MatMulGroup) continue;
      for (size_t m : l.members) moved_[m] = l.position;
    }
    for (size_t i = 0; i < steps_.size(); ++i) {
      if (taken_[i] || elided_[i] || Kind(i) != OpKind::Softmax) continue;
      auto it = readers_.find(steps_[i].out.name);
      if (it == readers_.end() || it->second.size() != 1) continue;
      const size_t j = it->second[0];
      size_t yi = fused->size();
      for (size_t k = 0; k < fused->size(); ++k) {
        const Launch &y = (*fused)[k];
        if (y.kind == Launch::Kind::MatMulChain && y.members[0] == j && y.group.empty() && !y.out.viewed) yi = k;
      }
      if (yi == fused->size()) continue;
      const std::vector<size_t> old_members = (*fused)[yi].members;
      for (size_t m : old_members) taken_[m] = false;
      std::optional<Launch> l = MatchSoftmaxMatVec(i);
      bool ok = l.has_value();
      for (size_t m : old_members) {
        ok = ok && std::find(l->members.begin(), l->members.end(), m) != l->members.end();
      }
      ok = ok && l->members.size() == old_members.size() + 1;
      for (size_t m : old_members) taken_[m] = true;
      if (!ok) continue;
      taken_[i] = true;
      (*fused)[yi] = std::move(*l);
    }
    moved_.clear();
    silent_.clear();
  }

  // Attention blocks the first sweep had to leave alone because a projection of the same block stood between
  // the score MatMul and the rest (the value projection after Q.K^T in the sequence): once GroupSiblings has moved
  // that projection in front, the block is matched again.  The contraction launches it overlaps are dissolved;
  // members the attention launch does not absorb go back to being single steps.
  void RetryAttention(std::vector<Launch> *fused) {
    moved_.assign(steps_.size(), SIZE_MAX);
    MarkSilent(*fused);
    for (const Launch &l : *fused) {
      if (l.kind != Launch::Kind::MatMulGroup) continue;
      for (size_t m : l.members) moved_[m] = l.position;
    }
    // launches an attention launch may take apart: contractions with their epilogues, and the Div -> Add -> Softmax
    // rows between the two products
    auto dissolvable = [](const Launch &y) {
      return y.kind == Launch::Kind::MatMulChain || y.kind == Launch::Kind::DivAddSoftmax;
    };
    // candidates for the score product: the head of a contraction launch, or a MatMul left as a single step
    for (size_t head = 0; head < steps_.size(); ++head) {
      if (Kind(head) != OpKind::MatMul || elided_[head]) continue;
      if (taken_[head]) {
        bool heads_chain = false;
        for (const Launch &x : *fused) heads_chain = heads_chain || (x.kind == Launch::Kind::MatMulChain && x.members[0] == head);
        if (!heads_chain) continue;
      }
      const std::vector<bool> saved = taken_;
      for (const Launch &y : *fused) {
        if (!dissolvable(y)) continue;
        for (size_t m : y.members) taken_[m] = false;
      }
      std::optional<Launch> l = MatchAttention(head);
      taken_ = saved;
      if (!l) continue;
      std::vector<size_t> touched;
      bool ok = true;
      size_t absorbed_free = 0, leftovers = 0;
      for (size_t m : l->members) {
        bool found = false;
        for (size_t yi = 0; yi < fused->size(); ++yi) {
          const Launch &y = (*fused)[yi];
          if (std::find(y.members.begin(), y.members.end(), m) == y.members.end()) continue;
          found = true;
          if (!dissolvable(y)) ok = false;
          if (std::find(touched.begin(), touched.end(), yi) == touched.end()) touched.push_back(yi);
        }
        if (!found) {
          if (taken_[m]) ok = false;
          ++absorbed_free;
        }
      }
      if (!ok) continue;
      for (size_t yi : touched) {
        for (size_t m : (*fused)[yi].members) {
          if (std::find(l->members.begin(), l->members.end(), m) == l->members.end()) ++leftovers;
        }
      }
      if (1 + leftovers >= touched.size() + absorbed_free) continue;  // no launch saved
      for (size_t yi : touched) {
        for (size_t m : (*fused)[yi].members) taken_[m] = false;
      }
      for (size_t m : l->members) taken_[m] = true;
      std::vector<Launch> kept;
      for (size_t yi = 0; yi < fused->size(); ++yi) {
        if (std::find(touched.begin(), touched.end(), yi) == touched.end()) kept.push_back(std::move((*fused)[yi]));
      }
      kept.push_back(std::move(*l));
      *fused = std::move(kept);
      MarkSilent(*fused);
    }
    moved_.clear();
    silent_.clear();
  }

  // scores = MatMul(q, k^T) -> Div | Mul by a constant [-> + mask] [-> Where(cond, x, fill)] -> Softmax over
  // the keys -> MatMul(p, v), optionally followed by the head-merging Transpose / Reshape: one launch that
  // keeps the score rows on chip.  The kernel's limits (head size, number of keys) are checked here so that
  // the launch can never be refused at replay time.
  std::optional<Launch> MatchAttention(size_t i) {
    const Step &scores = steps_[i];
    const auto &shape = scores.out.meta.GetShape();
    const auto &qs = scores.in0.meta.GetShape(), &ks = scores.in1.meta.GetShape();
    const size_t rank = shape.size();
    if (!IsFloat(scores.out) || rank < 2 || qs.size() != rank || ks.size() != rank) return std::nullopt;
    if (!std::equal(shape.begin(), shape.end() - 2, qs.begin()) || !std::equal(shape.begin(), shape.end() - 2, ks.begin())) {
      return std::nullopt;  // broadcast batch dims
    }
    const int64_t head = qs[rank - 1], keys = shape[rank - 1];
    if (head > 64 || keys > 256 || head == 0 || keys == 0) return std::nullopt;
    Launch l;
    l.kind = Launch::Kind::Attention;
    l.a = scores.in0;
    l.b = scores.in1;
    l.members = {i};
    std::vector<std::pair<size_t, Operand>> external = {{i, l.a}, {i, l.b}};
    auto next = SoleReader(i);
    if (!next || !IsFloat(steps_[*next].out) || steps_[*next].out.meta.GetShape() != shape) return std::nullopt;
    if (Kind(*next) == OpKind::DivConstantRhs) l.divisor = true;
    else if (Kind(*next) != OpKind::MulConstant) return std::nullopt;
    l.s0 = Attrs(*next).value;
    l.members.push_back(*next);
    size_t cur = *next;
    next = SoleReader(cur);
    if (next && Kind(*next) == OpKind::AddCommon && steps_[*next].out.meta.GetShape() == shape) {
      const auto mask = Other(*next, steps_[cur].out);
      if (!mask || !IsFloat(*mask)) return std::nullopt;
      l.d = *mask;
      l.has_mask = true;
      external.push_back({*next, l.d});
      l.members.push_back(*next);
      cur = *next;
      next = SoleReader(cur);
    }
    if (next && Kind(*next) == OpKind::WhereConstantCondConstantScalarY && IsFloat(steps_[*next].out) &&
        steps_[*next].out.meta.GetShape() == shape) {
      l.has_cond = true;
      l.owner = *next;
      l.s1 = Attrs(*next).value;
      l.members.push_back(*next);
      cur = *next;
      next = SoleReader(cur);
    }
    if (!next || Kind(*next) != OpKind::Softmax || steps_[*next].out.meta.GetShape() != shape) return std::nullopt;
    const int64_t axis = steps_[*next].node->GetAxis();
    if (axis != static_cast<int64_t>(rank) - 1 && axis != -1) return std::nullopt;
    l.members.push_back(*next);
    const Operand &probs = steps_[*next].out;
    next = SoleReader(*next);
    if (!next || Kind(*next) != OpKind::MatMul || !SameTensor(steps_[*next].in0, probs) || SameTensor(steps_[*next].in1, probs)) {
      return std::nullopt;
    }
    const size_t pv = *next;
    l.c = steps_[pv].in1;
    const auto &vs = l.c.meta.GetShape();
    if (!IsFloat(steps_[pv].out) || vs.size() != rank || !std::equal(shape.begin(), shape.end() - 2, vs.begin()) ||
        vs[rank - 1] != head) {
      return std::nullopt;
    }
    external.push_back({pv, l.c});
    l.members.push_back(pv);
    // `with_moves`: operands or a result the plan has other tenants for in the launch's window may move out of the
    // arena.  Tried only where nothing works without: a tensor in a buffer of its own costs the replayed graph a
    // little (BERT-base: 1 % with its twelve attention outputs moved for no launch less).
    auto finish = [&](Launch *x, bool with_moves) {
      std::vector<std::string> moves;
      const bool clash = !OutputDisjoint(x->out, {&x->a, &x->b, &x->c}) || (x->has_mask && Alias(x->out, x->d));
      if (clash && (!with_moves || !Movable(x->out))) return false;
      if (with_moves ? !SafeWithMoves(x->members, external, &moves) : !Safe(x->members, external)) return false;
      if (clash) moves.push_back(x->out.name);
      pending_moves_.insert(pending_moves_.end(), moves.begin(), moves.end());
      x->bytes = x->has_mask ? Bytes({&x->a, &x->b, &x->c, &x->d, &x->out}) : Bytes({&x->a, &x->b, &x->c, &x->out});
      if (x->has_cond) x->bytes += static_cast<double>(steps_[x->owner].kernel->GetConstantBytes());
      x->flops = Flops(x->members);
      return true;
    };
    for (const bool with_moves : {false, true}) {
      for (size_t limit = SIZE_MAX; limit > 0;) {
        Launch with_views = l;
        const size_t taken = AppendViews(pv, &with_views, limit);
        if (taken == 0) break;
        if (with_views.n_inner == 0 && finish(&with_views, with_moves)) return with_views;
        limit = taken - 1;
      }
    }
    l.out = steps_[pv].out;
    if (finish(&l, false) || finish(&l, true)) return l;
    return std::nullopt;
  }

  std::optional<Launch> MatchLayerNorm(size_t i) {
    const Step &add = steps_[i];
    if (!IsFloat(add.out)) return std::nullopt;
    if (add.in0.meta.GetShape() != add.out.meta.GetShape()) return std::nullopt;  // rhs may broadcast, lhs may not
    const auto j = SoleReader(i);
    if (!j || Kind(*j) != OpKind::LayerNormalizationConstantScaleBias) return std::nullopt;
    Launch l;
    l.kind = Launch::Kind::AddLayerNorm;
    l.members = {i, *j};
    l.a = add.in0;
    l.b = add.in1;
    l.out = steps_[*j].out;
    l.axis = Attrs(*j).axis;
    l.s0 = Attrs(*j).epsilon;
    l.owner = *j;
    if (!Safe(l.members, {{i, l.a}, {i, l.b}})) return std::nullopt;
    if (Alias(l.out, l.a) || Alias(l.out, l.b)) return std::nullopt;
    l.bytes = Bytes({&l.a, &l.b, &l.out}) + static_cast<double>(steps_[*j].kernel->GetConstantBytes());
    return l;
  }

  // ---- LayerNormalizations that never reach memory -------------------------------------------------------
  // AddCommon -> LayerNormalization behind a contraction (the post-attention and post-FFN normalisations of a
  // transformer layer) costs a launch of its own that moves 1 MB and takes 4.5 us of pure latency.  Instead:
  //   * the contraction in front absorbs the AddCommon (the residual becomes its addend) and, where the normalised
  //     tensor h has no reader that needs it in memory, the LayerNormalization too: it stores the sum s in h's buffer
  //     and leaves partial row statistics of s in a private buffer;
  //   * every reader of h is then a contraction that takes h as its left operand -- it multiplies s with the scale
  //     folded into its weights and applies mean and 1/sigma per row in its epilogue -- or the AddCommon of the next
  //     such pair, whose contraction normalises s while adding it.
  // Decided back to front: a LayerNormalization can only stay out of memory if the pair that reads it as a residual
  // can absorb its AddCommon.  A pair whose residual is such a tensor but whose own result has to exist (a graph
  // output, or a reader that is neither of the above) absorbs the AddCommon only and runs its LayerNormalization as
  // a step.  Launch positions: the widened launch runs where its last member stood, so its late reads and the early
  // use of h's buffer go through the same checks as every other chain.
  void DeferLayerNorms(std::vector<Launch> *fused) {
    if (const char *v = std::getenv("FLUIDML_DEFER_NORM"); v != nullptr && std::string(v) == "0") return;
    std::vector<int> owner(steps_.size(), -1);
    for (size_t k = 0; k < fused->size(); ++k) {
      for (size_t m : (*fused)[k].members) owner[m] = static_cast<int>(k);
    }
    std::vector<size_t> norms;
    for (size_t k = 0; k < fused->size(); ++k) {
      if ((*fused)[k].kind == Launch::Kind::AddLayerNorm) norms.push_back(k);
    }
    std::sort(norms.begin(), norms.end(), [&](size_t x, size_t y) { return (*fused)[x].members.back() < (*fused)[y].members.back(); });
    struct Decision {
      int producer = -1;  // launch that computes one addend of the AddCommon and can take the other as its addend
      Operand residual;   // that other addend
      bool absorbable = false;  // the launch can take the AddCommon, one way or the other:
      bool sum_in_place = false;  // ... writing the sum where the plan put it (the LayerNormalization then runs as a step)
      bool deferrable = false;    // ... or taking the LayerNormalization too (every reader normalises on the fly)
      bool relocate = false;      // deferrable, but the plan put the normalised tensor over bytes the launch still reads
    };
    std::map<size_t, Decision> decisions;
    std::vector<bool> produces(fused->size(), false);  // launches an (already decided, later) pair would widen
    auto one_row_block = [](const std::vector<int64_t> &shape) {
      int64_t batch = 1;
      for (size_t d = 0; d + 2 < shape.size(); ++d) batch *= shape[d];
      return shape.size() >= 2 && batch == 1;
    };
    // `m` (a MatMulChain, alone or inside a group) multiplies h from the left by a constant matrix only it reads
    auto takes_as_lhs = [&](const Launch &m, size_t reader, const Operand &h, int64_t width) {
      if (m.kind != Launch::Kind::MatMulChain || m.members[0] != reader || Kind(reader) != OpKind::MatMul) return false;
      if (!SameTensor(m.a, h) || m.a.viewed || !SameTensor(steps_[reader].in0, h) || m.has_skip || m.norm_mode != 0) return false;
      const Operand &w = m.b;
      if (w.space != Operand::Space::Constant || w.viewed || !IsFloat(w) || !DefaultLayout(w)) return false;
      const auto &wshape = w.meta.GetShape();
      if (wshape.size() != 2 || wshape[0] != width) return false;
      const auto it = readers_.find(w.name);
      if (it == readers_.end() || it->second.size() != 1) return false;  // the weights get the scale folded in
      return !m.has_c || (m.c.space == Operand::Space::Constant && m.c.meta.GetShape().size() == 1);
    };
    for (auto it = norms.rbegin(); it != norms.rend(); ++it) {
      const size_t k = *it;
      const Launch &pair = (*fused)[k];
      const size_t add = pair.members[0], ln = pair.members[1];
      const auto &shape = pair.out.meta.GetShape();
      Decision dec;
      if (!IsFloat(pair.out) || !one_row_block(shape)) {
        decisions[k] = dec;
        continue;
      }
      for (int side = 0; side < 2 && !dec.absorbable; ++side) {
        const Operand &y = side == 0 ? pair.a : pair.b, &x = side == 0 ? pair.b : pair.a;
        if (y.viewed || x.viewed || !Elidable(y) || !DefaultLayout(y) || !DefaultLayout(x) || !IsFloat(x)) continue;
        if (x.space == Operand::Space::Constant || x.meta.GetShape() != shape || y.meta.GetShape() != shape) continue;
        const auto made = producer_.find(y.name);
        if (made == producer_.end() || owner[made->second] < 0) continue;
        const auto yr = readers_.find(y.name);
        if (yr == readers_.end() || yr->second.size() != 1 || yr->second[0] != add) continue;
        const Launch &p = (*fused)[static_cast<size_t>(owner[made->second])];
        if (p.kind != Launch::Kind::MatMulChain || p.has_skip || !p.view_strides.empty() || p.n_inner != 0 || p.norm_mode != 0 ||
            !SameTensor(p.out, y) || p.out.viewed || p.members.back() != made->second) {
          continue;
        }
        if (!IsFloat(p.b) || p.b.viewed || !DefaultLayout(p.b) || p.b.meta.GetShape().size() != 2) continue;
        std::vector<size_t> members = p.members;
        members.push_back(add);
        const std::vector<std::pair<size_t, Operand>> external = {{p.members[0], p.a}, {p.members[0], p.b}, {add, x}};
        const Operand &sum = steps_[add].out;
        if (!DefaultLayout(sum) || sum.viewed) continue;  // (the addend is read with the strides of what the launch writes)
        if (!Safe(members, external)) continue;
        dec.producer = owner[made->second];
        dec.residual = x;
        dec.sum_in_place = OutputDisjoint(sum, {&p.a, &p.b}) && !Alias(sum, x);
        dec.absorbable = true;  // (unless neither form works out below)
      }
      if (dec.absorbable) {
        const Launch &p = (*fused)[static_cast<size_t>(dec.producer)];
        const int64_t rank = static_cast<int64_t>(shape.size());
        const int64_t axis = pair.axis < 0 ? pair.axis + rank : pair.axis;
        const kernel::Kernel &norm = *steps_[ln].kernel;
        bool ok = axis == rank - 1 && shape.back() <= 1024 && Elidable(pair.out) && !pair.out.viewed && DefaultLayout(pair.out) &&
                  norm.GetConstant(0) != nullptr && norm.GetConstant(1) != nullptr && Attrs(ln).t0 && Attrs(ln).t1;
        std::vector<size_t> members = p.members;
        members.push_back(add);
        members.push_back(ln);
        ok = ok && Safe(members, {{p.members[0], p.a}, {p.members[0], p.b}, {add, dec.residual}});
        // The plan often reuses the bytes of the contraction's left operand for what comes behind it.  The launch
        // reads while it writes, so the tensor then goes into a buffer of its own, outside the arena, like what a
        // side branch writes: the plan's offsets stay as they are, the bytes are reported as private.
        dec.relocate = !(OutputDisjoint(pair.out, {&p.a, &p.b}) && !Alias(pair.out, dec.residual));
        const auto hr = readers_.find(pair.out.name);
        ok = ok && hr != readers_.end() && !hr->second.empty();
        for (size_t r : (ok ? hr->second : std::vector<size_t>{})) {
          if (owner[r] < 0) {
            ok = false;
            break;
          }
          const size_t c = static_cast<size_t>(owner[r]);
          const Launch &reader = (*fused)[c];
          bool fine = false;
          if (reader.kind == Launch::Kind::AddLayerNorm) {
            const auto d = decisions.find(c);
            fine = reader.members[0] == r && d != decisions.end() && d->second.absorbable && SameTensor(d->second.residual, pair.out);
          } else if (reader.kind == Launch::Kind::MatMulChain) {
            // (a launch takes one deferred operand: not the left one if it may get a deferred residual later)
            fine = !produces[c] && takes_as_lhs(reader, r, pair.out, shape.back());
          } else if (reader.kind == Launch::Kind::MatMulGroup) {
            for (const Launch &m : reader.group) fine = fine || takes_as_lhs(m, r, pair.out, shape.back());
          }
          ok = ok && fine;
        }
        dec.deferrable = ok;
        dec.absorbable = dec.deferrable || dec.sum_in_place;
        if (dec.absorbable) produces[static_cast<size_t>(dec.producer)] = true;
      }
      decisions[k] = dec;
    }
    std::map<std::string, size_t> deferred;  // normalised tensors that stay out of memory -> their LayerNormalization step
    std::map<std::string, Operand> moved;    // ... and where they live, if not where the plan put them
    std::vector<bool> drop(fused->size(), false);
    for (size_t k : norms) {
      const Decision &dec = decisions[k];
      if (!dec.absorbable) continue;
      const Launch pair = (*fused)[k];
      const size_t add = pair.members[0], ln = pair.members[1];
      const auto from = deferred.find(dec.residual.name);
      const bool residual_deferred = from != deferred.end() && dec.residual.space != Operand::Space::Constant;
      if (!dec.deferrable && !residual_deferred) continue;  // the pair stays one AddLayerNorm launch
      Launch wide = (*fused)[static_cast<size_t>(dec.producer)];
      wide.members.push_back(add);
      const auto at = moved.find(dec.residual.name);
      wide.d = residual_deferred && at != moved.end() ? at->second : dec.residual;
      wide.has_skip = true;
      wide.bytes += static_cast<double>(dec.residual.meta.GetSize());
      if (residual_deferred) {
        wide.norm_mode = 2;
        wide.norm_owner = from->second;
        wide.norm_stats = "norm:" + dec.residual.name;
      }
      if (dec.deferrable) {
        wide.members.push_back(ln);
        wide.out = pair.out;
        if (dec.relocate) {
          wide.out.space = Operand::Space::Private;
          wide.out.offset = 0;
          wide.out.pool.clear();
          moved[pair.out.name] = wide.out;
        }
        wide.norm_stats_out = "norm:" + pair.out.name;
        deferred[pair.out.name] = ln;
      } else {
        wide.out = steps_[add].out;
        taken_[ln] = false;  // the LayerNormalization runs as a step of its own, on the sum the launch wrote
      }
      wide.flops = Flops(wide.members);
      (*fused)[k] = wide;
      drop[static_cast<size_t>(dec.producer)] = true;
      if (!dec.deferrable) continue;
      for (size_t r : readers_.at(pair.out.name)) {
        Launch &reader = (*fused)[static_cast<size_t>(owner[r])];
        if (reader.kind == Launch::Kind::AddLayerNorm) continue;  // widened when its turn comes
        reader.norm_mode = 1;
        reader.norm_owner = ln;
        reader.norm_stats = "norm:" + pair.out.name;
        if (dec.relocate) {
          reader.a = wide.out;
          for (Launch &m : reader.group) m.a = wide.out;
        }
      }
    }
    std::vector<Launch> kept;
    for (size_t k = 0; k < fused->size(); ++k) {
      if (!drop[k]) kept.push_back(std::move((*fused)[k]));
    }
    *fused = std::move(kept);
    DeferLoneLayerNorms(fused);
  }

  // The pre-norm form (GPT-style blocks): x, written by a contraction launch (the residual sum of the block in front),
  // goes through a LayerNormalization of its own whose result only feeds contractions as their left operand.  The
  // launch that writes x also leaves its partial row statistics, the LayerNormalization does not run, and its readers
  // take x itself and normalise on the fly (the FL_NORM_LHS form above; several LayerNormalizations of one x -- the two
  // of a parallel-residual block -- each fold their own scale and shift into their readers' weights).  For the
  // schedule the step becomes a view of x, with everything that guards a view: x's bytes must stay untouched until
  // the last of these readers has run, else x moves to a buffer of its own.
  void DeferLoneLayerNorms(std::vector<Launch> *fused) {
    for (size_t i = 0; i < steps_.size(); ++i) {
      if (Kind(i) != OpKind::LayerNormalizationConstantScaleBias || taken_[i] || elided_[i]) continue;
      std::vector<int> owner(steps_.size(), -1);  // (rebuilt per step: the list does not change here, but stays cheap)
      for (size_t k = 0; k < fused->size(); ++k) {
        for (size_t m : (*fused)[k].members) owner[m] = static_cast<int>(k);
      }
      const Step &ln = steps_[i];
      const Operand x = ln.in0, h = ln.out;
      const auto &shape = h.meta.GetShape();
      const int64_t rank = static_cast<int64_t>(shape.size());
      int64_t batch = 1;
      for (size_t d = 0; d + 2 < shape.size(); ++d) batch *= shape[d];
      const int64_t axis = Attrs(i).axis < 0 ? Attrs(i).axis + rank : Attrs(i).axis;
      if (rank < 2 || batch != 1 || axis != rank - 1 || shape.back() > 1024 || !IsFloat(h) || !IsFloat(x)) continue;
      if (x.viewed || h.viewed || !Elidable(h) || !DefaultLayout(h) || !DefaultLayout(x) || x.meta.GetShape() != shape) continue;
      if (ln.kernel->GetConstant(0) == nullptr || ln.kernel->GetConstant(1) == nullptr || !Attrs(i).t0 || !Attrs(i).t1) continue;
      // who writes x
      const auto made = producer_.find(x.name);
      if (made == producer_.end()) continue;
      const std::string stats = "norm:" + x.name;
      // an embedding lookup that runs as a step of its own can leave the statistics as well (GatherStats)
      const bool from_lookup = owner[made->second] < 0;
      if (from_lookup) {
        const size_t g = made->second;
        if (Kind(g) != OpKind::GatherConstantDataTensor || taken_[g] || elided_[g] || !SameTensor(steps_[g].out, x) ||
            steps_[g].kernel->GetConstant(0) == nullptr || steps_[g].in0.viewed || !DefaultLayout(steps_[g].in0) ||
            static_cast<int64_t>(steps_[g].in0.meta.GetShape().size()) != rank - 1 || g >= i) {
          continue;
        }
      } else {
        const Launch &p = (*fused)[static_cast<size_t>(owner[made->second])];
        if (p.kind == Launch::Kind::GatherStats) {
          if (p.norm_stats_out != stats) continue;
        } else {
          if (p.kind != Launch::Kind::MatMulChain || !p.group.empty() || !SameTensor(p.out, x) || p.out.viewed ||
              !p.view_strides.empty() || p.n_inner != 0 || p.members.back() != made->second) {
            continue;
          }
          if (!IsFloat(p.b) || p.b.viewed || !DefaultLayout(p.b) || p.b.meta.GetShape().size() != 2) continue;
          if (!p.norm_stats_out.empty() && p.norm_stats_out != stats) continue;
        }
      }
      // who reads the normalised tensor
      const auto hr = readers_.find(h.name);
      if (hr == readers_.end() || hr->second.empty()) continue;
      bool ok = true;
      std::vector<size_t> reader_launches;
      size_t last_position = i;
      for (size_t r : hr->second) {
        if (owner[r] < 0) {
          ok = false;
          break;
        }
        const size_t c = static_cast<size_t>(owner[r]);
        const Launch &reader = (*fused)[c];
        bool fine = false;
        auto lhs_of = [&](const Launch &m) {
          if (m.kind != Launch::Kind::MatMulChain || m.members[0] != r || Kind(r) != OpKind::MatMul) return false;
          if (!SameTensor(m.a, h) || m.a.viewed || !SameTensor(steps_[r].in0, h) || m.norm_mode != 0) return false;
          const Operand &w = m.b;
          if (w.space != Operand::Space::Constant || w.viewed || !IsFloat(w) || !DefaultLayout(w)) return false;
          const auto &wshape = w.meta.GetShape();
          if (wshape.size() != 2 || wshape[0] != shape.back()) return false;
          const auto wr = readers_.find(w.name);
          if (wr == readers_.end() || wr->second.size() != 1) return false;  // the weights get the scale folded in
          return !m.has_c || (m.c.space == Operand::Space::Constant && m.c.meta.GetShape().size() == 1);
        };
        if (reader.kind == Launch::Kind::MatMulChain) {
          fine = !reader.has_skip && lhs_of(reader);  // (with an addend the launch may still get a deferred residual)
        } else if (reader.kind == Launch::Kind::MatMulGroup) {
          for (const Launch &m : reader.group) fine = fine || lhs_of(m);
        }
        ok = ok && fine && !Alias(reader.out, x);
        for (const Launch &m : reader.group) ok = ok && !Alias(m.out, x);
        const size_t pos = reader.kind == Launch::Kind::MatMulGroup ? reader.position : reader.members.back();
        ok = ok && pos > i;
        last_position = std::max(last_position, pos);
        if (std::find(reader_launches.begin(), reader_launches.end(), c) == reader_launches.end()) reader_launches.push_back(c);
      }
      if (!ok) continue;
      // x's bytes between the LayerNormalization and the last of its readers: anything issued in between that
      // writes them (outputs of single steps at their own place, of launches at the place they are issued)
      bool untouched = true;
      for (size_t s = i + 1; s < last_position && untouched; ++s) {
        if (owner[s] < 0 && !elided_[s] && Alias(steps_[s].out, x)) untouched = false;
      }
      for (const Launch &l : *fused) {
        const size_t pos = l.kind == Launch::Kind::MatMulGroup ? l.position : l.members.back();
        if (pos <= i || pos >= last_position) continue;
        if (l.group.empty() && Alias(l.out, x)) untouched = false;
        if (l.has_out2 && Alias(l.out2, x)) untouched = false;
        for (const Launch &m : l.group) untouched = untouched && !Alias(m.out, x);
      }
      if (!untouched) {
        if (!Movable(x)) continue;
        MoveOut(x.name, {fused});
      }
      const Operand source = steps_[i].in0;  // (x, where it lives now)
      if (from_lookup) {
        const size_t g = made->second;
        Launch lookup;
        lookup.kind = Launch::Kind::GatherStats;
        lookup.members = {g};
        lookup.a = steps_[g].in0;
        lookup.out = steps_[g].out;
        lookup.owner = g;
        lookup.bytes = steps_[g].bytes;
        lookup.norm_stats_out = stats;
        taken_[g] = true;
        fused->push_back(std::move(lookup));
      } else {
        (*fused)[static_cast<size_t>(owner[made->second])].norm_stats_out = stats;
      }
      for (size_t c : reader_launches) {
        Launch &reader = (*fused)[c];
        reader.norm_mode = 1;
        reader.norm_owner = i;
        reader.norm_stats = stats;
        if (SameTensor(reader.a, h)) reader.a = source;
        for (Launch &m : reader.group) {
          if (SameTensor(m.a, h)) m.a = source;
        }
      }
      for (size_t r : hr->second) {
        steps_[r].in0 = source;
        rewired_[r] = true;
      }
      steps_[i].out = source;  // the step is a view of x now: nothing runs, nothing is written
      steps_[i].out.meta = h.meta;
      steps_[i].out.viewed = true;
      steps_[i].out.view_offset = 0;
      steps_[i].out.view_strides = LogicalStrides(source);
      steps_[i].out.source_bytes = source.Extent();
      elided_[i] = true;
      taken_[i] = true;
      BuildReaders();
    }
  }

  // Pad (constant zero) whose result only goes through steps that re-address it -- Gather with sliding-window
  // indices, Slice, Transpose, Reshape, each the only reader of the one before -- until the last of them: one copy
  // that reads the Pad's input and writes the last step's output; the padded tensor and the views are never written.
  std::optional<Launch> MatchPadViewCopy(size_t i) {
    const Step &pad = steps_[i];
    if (pad.in0.meta.GetType() != Type::kFloat32 || pad.in0.viewed || !DefaultLayout(pad.out)) return std::nullopt;
    const auto &pshape = pad.out.meta.GetShape();
    if (Attrs(i).pad_pairs.size() != pshape.size()) return std::nullopt;
    Launch l;
    l.kind = Launch::Kind::PadViewCopy;
    l.members = {i};
    l.a = pad.in0;
    Operand cur = pad.out;  // what the next step reads, as a view of the padded tensor
    std::optional<Launch> best;
    size_t at = i;
    while (true) {
      const auto j = SoleReader(at);
      if (!j || !steps_[*j].node->IsSingleInput() || !SameTensor(steps_[*j].in0, steps_[at].out)) break;
      // the step's input: the padded tensor itself, then the previous view step's output seen inside it
      const auto view = AsViewOf(*j, at == i ? pad.out : cur);
      if (!view) break;
      Operand seen = steps_[*j].out;
      seen.space = pad.out.space;
      seen.name = pad.out.name;
      seen.offset = pad.out.offset;
      seen.viewed = true;
      seen.view_offset = view->first;
      seen.view_strides = view->second;
      seen.source_bytes = pad.out.meta.GetSize();
      cur = seen;
      l.members.push_back(*j);
      at = *j;
      // a launch that ends here: the view materialised into this step's own output
      Launch candidate = l;
      candidate.out = steps_[at].out;
      candidate.view_offset = view->first;
      candidate.view_strides = view->second;
      if (candidate.members.size() >= 3 && Elidable(steps_[at].out) && Safe(candidate.members, {{i, l.a}}) &&
          !Alias(candidate.out, l.a)) {
        candidate.bytes = Bytes({&l.a, &candidate.out});
        best = candidate;
      }
    }
    return best;
  }

  std::optional<Launch> MatchCopyPair(size_t i, OpKind second) {
    const auto j = SoleReader(i);
    if (!j || Kind(*j) != second) return std::nullopt;
    Launch l;
    l.kind = second == OpKind::Transpose ? Launch::Kind::ReshapeTranspose : Launch::Kind::TransposeReshape;
    l.members = {i, *j};
    l.a = steps_[i].in0;
    l.out = steps_[*j].out;
    l.perm = Attrs(second == OpKind::Transpose ? *j : i).perm;
    if (!Safe(l.members, {{i, l.a}}) || Alias(l.out, l.a)) return std::nullopt;
    l.bytes = Bytes({&l.a, &l.out});
    return l;
  }

  std::vector<Step> steps_;  // own copy: view elision rewrites the inputs of the readers
  std::vector<bool> taken_, elided_, rewired_;
  std::vector<std::string> pending_moves_;  // results to move out of the arena when the matching sweeps are over
  std::vector<bool> silent_;   // per step: an intermediate of a fused launch, never written (filled by RetryAttention)
  std::vector<size_t> moved_;  // per step: the position its launch is issued at when a group moved it (else SIZE_MAX)
  std::vector<int> placed_;  // Concat2 steps: bit 0 / 1 = input 0 / 1 is written in place by its producer
  std::vector<bool> filled_;  // Reshape steps whose buffer the Concat2 in front of them wrote: nothing runs
  std::unordered_map<std::string, std::vector<size_t>> readers_;
  std::unordered_map<std::string, size_t> producer_;  // tensor name -> the step that writes it
};

}  // namespace

std::vector<Launch> BuildSchedule(const std::vector<Step> &steps, bool fuse) { return Scheduler(steps).Run(fuse); }

}  // namespace worker
}  // namespace fluidml
