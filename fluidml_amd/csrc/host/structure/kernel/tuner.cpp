#include "structure/kernel/tuner.h"

#include <cstdlib>
#include <fstream>
#include <limits>
#include <sstream>
#include <stdexcept>

namespace fluidml {
namespace kernel {

ContractionTable ContractionTable::FromEnvironment() {
  const char *v = std::getenv("FLUIDML_TUNE");
  if (v == nullptr || std::string(v) == "1" || std::string(v).empty()) return ContractionTable(Mode::Measure);
  if (std::string(v) == "0") return ContractionTable(Mode::Off);
  std::ifstream ifs(v);
  if (!ifs) throw std::runtime_error(std::string("FLUIDML_TUNE: cannot open ") + v);
  std::stringstream text;
  text << ifs.rdbuf();
  ContractionTable table(Mode::Replay);
  table.LoadJsonText(text.str());
  return table;
}

bool ContractionTable::Find(const std::string &signature, ContractPick *pick) const {
  auto it = picks_.find(signature);
  if (it == picks_.end()) return false;
  if (pick != nullptr) *pick = it->second;
  return true;
}

void ContractionTable::Put(const std::string &signature, const ContractPick &pick) { picks_[signature] = pick; }

std::string ContractionTable::ToJson() const {
  std::ostringstream os;
  os << "{";
  bool first = true;
  for (const auto &kv : picks_) {
    os << (first ? "" : ",") << json::Quote(kv.first) << ":{\"tile\":" << kv.second.tile << ",\"splits\":" << kv.second.splits
       << ",\"ns\":" << static_cast<long long>(kv.second.ns) << ",\"rule_ns\":" << static_cast<long long>(kv.second.rule_ns)
       << "}";
    first = false;
  }
  os << "}";
  return os.str();
}

void ContractionTable::LoadJson(const json::Value &doc) {
  const json::Value &table = doc.Has("contraction_table") ? doc.At("contraction_table") : doc;
  if (table.kind != json::Value::Kind::Object) throw std::runtime_error("contraction table: not a JSON object");
  for (const auto &kv : table.object) {
    const json::Value &e = kv.second;
    if (!e.Has("tile") || !e.Has("splits")) continue;  // some other member of a larger document
    ContractPick pick;
    pick.tile = static_cast<int>(e.At("tile").number);
    pick.splits = static_cast<int>(e.At("splits").number);
    if (pick.tile < 0 || pick.tile >= FL_TILE_COUNT || pick.splits < 0 || pick.splits > FL_CONTRACT_MAX_SPLITS) {
      throw std::runtime_error("contraction table: entry '" + kv.first + "' names no tile configuration");
    }
    if (e.Has("ns")) pick.ns = e.At("ns").number;
    if (e.Has("rule_ns")) pick.rule_ns = e.At("rule_ns").number;
    picks_[kv.first] = pick;
  }
}

void ContractionTable::LoadJsonText(const std::string &text) { LoadJson(json::Parse(text)); }

std::vector<std::pair<int, int>> ContractionTable::Candidates(bool full) {
  std::vector<std::pair<int, int>> out;
  if (full) {
    for (int tile = 1; tile < FL_TILE_COUNT; ++tile) {
      for (int splits : {0, 1, 2, 3, 4, 6, 8, 12, 16}) out.push_back({tile, splits});
    }
  } else {
    for (int tile = 1; tile < FL_TILE_COUNT; ++tile) out.push_back({tile, 0});
    for (int splits : {1, 2, 4, 8}) out.push_back({FL_TILE_RULE, splits});
  }
  return out;
}

ContractPick ContractionTable::Measure(const std::vector<std::pair<int, int>> &candidates,
                                       const std::function<int(uint32_t)> &launch,
                                       const std::function<double()> &elapsed_ns, int rounds, double margin) {
  auto time_of = [&](const ContractPick &c, double *ns) {
    double best = std::numeric_limits<double>::max();
    for (int r = 0; r <= rounds; ++r) {  // round 0 warms up
      const int rc = launch(c.Flags());
      if (rc == FL_ERR_UNSUPPORTED) return false;
      if (rc != 0) throw std::runtime_error(std::string("timing a contraction: ") + fluidml_hip_error_string(rc));
      const double t = elapsed_ns();
      if (r > 0 && t < best) best = t;
    }
    *ns = best;
    return true;
  };
  ContractPick rule;
  if (!time_of(rule, &rule.ns)) throw std::runtime_error("timing a contraction: the library's rule refuses the problem");
  rule.rule_ns = rule.ns;
  ContractPick best = rule;
  for (const auto &c : candidates) {
    ContractPick p;
    p.tile = c.first;
    p.splits = c.second;
    p.rule_ns = rule.ns;
    if (!time_of(p, &p.ns)) continue;
    const double bar = best.IsRule() ? rule.ns * (1.0 - margin) : best.ns;
    if (p.ns < bar) best = p;
  }
  return best;
}

std::string ContractionTable::Signature(const std::string &kind, const fl_tensor &lhs, const fl_tensor &rhs,
                                        const fl_tensor &out, int group, const std::string &epilogue) {
  std::ostringstream os;
  auto view = [&](const fl_tensor &t) {
    os << "[";
    for (int32_t i = 0; i < t.rank; ++i) os << (i ? "," : "") << t.shape[i];
    os << "](";
    for (int32_t i = 0; i < t.rank; ++i) os << (i ? "," : "") << t.strides[i];
    os << ")" << (reinterpret_cast<uintptr_t>(t.base) % 16 == 0 ? "a" : "u");
  };
  os << kind << " ";
  view(lhs);
  os << "x";
  view(rhs);
  os << "->";
  view(out);
  os << " g" << group << " " << epilogue;
  return os.str();
}

}  // namespace kernel
}  // namespace fluidml
