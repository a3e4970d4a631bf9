// Launch-level fusion: groups the steps of a launch plan into chains that one
// HIP kernel computes.  The node sequence, the memory plan and every tensor a
// later step (or the caller) can observe stay exactly as planned; only tensors
// with a single reader inside a chain are no longer written.  The reference
// fuses at graph level before planning (e.g. its AddDivErfAddMulMul node,
// src/structure/flow/node.cpp); it has no counterpart of this pass because it
// pays no per-kernel launch cost.
#include <algorithm>
#include <optional>
#include <unordered_map>

#include "worker/launcher.h"

namespace fluidml {
namespace worker {

const char *LaunchKindName(Launch::Kind kind) {
  switch (kind) {
    case Launch::Kind::Step: return "Step";
    case Launch::Kind::MatMulAdd: return "MatMulAdd";
    case Launch::Kind::MatMulAddGelu: return "MatMulAddDivErfAddMulMul";
    case Launch::Kind::DivAddSoftmax: return "DivAddSoftmax";
    case Launch::Kind::AddLayerNorm: return "AddLayerNormalization";
    case Launch::Kind::ReshapeTranspose: return "ReshapeTranspose";
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
  const size_t x1 = x.offset + x.meta.GetSize(), y1 = y.offset + y.meta.GetSize();
  return x.offset < y1 && y.offset < x1;
}

bool IsFloat(const Operand &o) { return o.meta.GetType() == Type::kFloat32; }

class Scheduler {
 public:
  Scheduler(const std::vector<Step> &steps) : steps_(steps), taken_(steps.size(), false) {
    for (size_t i = 0; i < steps_.size(); ++i) {
      const Step &s = steps_[i];
      readers_[s.in0.name].push_back(i);
      if (s.node->IsDoubleInputs() && !SameTensor(s.in0, s.in1)) readers_[s.in1.name].push_back(i);
    }
  }

  std::vector<Launch> Run(bool fuse) {
    std::vector<Launch> fused;
    if (fuse) {
      for (size_t i = 0; i < steps_.size(); ++i) {
        if (taken_[i]) continue;
        std::optional<Launch> l;
        switch (Kind(i)) {
          case OpKind::MatMul: l = MatchMatMul(i); break;
          case OpKind::DivConstantRhs: l = MatchSoftmax(i); break;
          case OpKind::AddCommon: l = MatchLayerNorm(i); break;
          case OpKind::Reshape: l = MatchCopyPair(i, OpKind::Transpose); break;
          case OpKind::Transpose: l = MatchCopyPair(i, OpKind::Reshape); break;
          default: break;
        }
        if (l) {
          for (size_t m : l->members) taken_[m] = true;
          fused.push_back(std::move(*l));
        }
      }
    }
    // a chain is issued where its last member stood; everything else keeps its place
    std::vector<const Launch *> at(steps_.size(), nullptr);
    for (const Launch &l : fused) at[l.members.back()] = &l;
    std::vector<Launch> schedule;
    for (size_t i = 0; i < steps_.size(); ++i) {
      if (at[i] != nullptr) {
        schedule.push_back(*at[i]);
      } else if (!taken_[i]) {
        Launch l;
        l.members = {i};
        l.bytes = steps_[i].bytes;
        l.flops = steps_[i].flops;
        schedule.push_back(std::move(l));
      }
    }
    return schedule;
  }

 private:
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
        if (Alias(steps_[s].out, op)) return false;
      }
    }
    // the chain's own output must not overwrite an external input another member still needs: the fused kernel
    // reads and writes concurrently, the unfused sequence only tolerates that element for element
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

  std::optional<Launch> MatchMatMul(size_t i) {
    const Step &mm = steps_[i];
    if (!IsFloat(mm.out)) return std::nullopt;
    const auto j = SoleReader(i);
    if (!j || Kind(*j) != OpKind::AddCommon) return std::nullopt;
    const auto bias = Other(*j, mm.out);
    const Step &add = steps_[*j];
    if (!bias || bias->space != Operand::Space::Constant || !IsFloat(*bias)) return std::nullopt;
    const auto &shape = mm.out.meta.GetShape();
    if (bias->meta.GetShape().size() != 1 || bias->meta.GetShape()[0] != shape.back()) return std::nullopt;
    if (add.out.meta.GetShape() != shape) return std::nullopt;

    Launch l;
    l.a = mm.in0;
    l.b = mm.in1;
    l.c = *bias;
    // try to extend through the erf-GELU chain
    if (auto g = MatchGelu(*j)) {
      l.kind = Launch::Kind::MatMulAddGelu;
      l.members = {i, *j};
      l.members.insert(l.members.end(), g->members.begin(), g->members.end());
      l.out = steps_[l.members.back()].out;
      l.s0 = g->s0;
      l.s1 = g->s1;
      l.s2 = g->s2;
      if (Safe(l.members, {{i, l.a}, {i, l.b}}) && OutputDisjoint(l.out, {&l.a, &l.b})) {
        l.bytes = Bytes({&l.a, &l.b, &l.c, &l.out});
        l.flops = Flops(l.members);
        return l;
      }
    }
    l.kind = Launch::Kind::MatMulAdd;
    l.members = {i, *j};
    l.out = add.out;
    if (!Safe(l.members, {{i, l.a}, {i, l.b}}) || !OutputDisjoint(l.out, {&l.a, &l.b})) return std::nullopt;
    l.bytes = Bytes({&l.a, &l.b, &l.c, &l.out});
    l.flops = Flops(l.members);
    return l;
  }

  // t = steps[j].out; Div(t, c) -> Erf -> Add(c) -> Mul(t, .) -> Mul(c): members after j, scalars in s0..s2
  std::optional<Launch> MatchGelu(size_t j) const {
    const Operand &t = steps_[j].out;
    if (!Elidable(t)) return std::nullopt;
    auto it = readers_.find(t.name);
    if (it == readers_.end() || it->second.size() != 2) return std::nullopt;
    size_t d = it->second[0], m = it->second[1];
    if (Kind(d) != OpKind::DivConstantRhs) std::swap(d, m);
    if (Kind(d) != OpKind::DivConstantRhs || Kind(m) != OpKind::MulCommon) return std::nullopt;
    if (d <= j || taken_[d] || taken_[m]) return std::nullopt;
    const auto e = SoleReader(d);
    if (!e || Kind(*e) != OpKind::Erf) return std::nullopt;
    const auto a = SoleReader(*e);
    if (!a || Kind(*a) != OpKind::AddConstant) return std::nullopt;
    const auto m2 = SoleReader(*a);
    if (!m2 || *m2 != m) return std::nullopt;
    const auto other = Other(m, steps_[*a].out);
    if (!other || !SameTensor(*other, t)) return std::nullopt;
    const auto r = SoleReader(m);
    if (!r || Kind(*r) != OpKind::MulConstant) return std::nullopt;
    for (size_t s : {d, *e, *a, m, *r}) {
      if (steps_[s].out.meta.GetShape() != t.meta.GetShape() || !IsFloat(steps_[s].out)) return std::nullopt;
    }
    Launch l;
    l.members = {d, *e, *a, m, *r};
    if (!std::is_sorted(l.members.begin(), l.members.end())) return std::nullopt;
    l.s0 = Attrs(d).value;
    l.s1 = Attrs(*a).value;
    l.s2 = Attrs(*r).value;
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

  const std::vector<Step> &steps_;
  std::vector<bool> taken_;
  std::unordered_map<std::string, std::vector<size_t>> readers_;
};

}  // namespace

std::vector<Launch> BuildSchedule(const std::vector<Step> &steps, bool fuse) { return Scheduler(steps).Run(fuse); }

}  // namespace worker
}  // namespace fluidml
