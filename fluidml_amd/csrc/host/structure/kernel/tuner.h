// Which tile configuration each contraction of a graph runs with.
//
// The reference's MatMul and Gemm generators time the six loop orders of their kernel on filled buffers
// and cache the fastest one per (lhs, rhs, output) layout triple (src/structure/kernel/generator/matmul.cpp:88-131,
// gemm.cpp:106-151).  On this backend the loop order is fixed by the matrix-core instruction; what is worth
// choosing per problem is the workgroup tile and the number of workgroups that share a tile's K range
// (fl_contract_tile and the split count of include/fluidml_hip.h).  A ContractionTable holds that choice per
// problem signature -- extents, element strides (i.e. the layouts), 16-byte alignment of the operands, the number
// of grouped siblings and the epilogue -- filled by measurement at Compile, written into the executor's JSON
// beside the layout DP's cost table, and read back from such a file so that a later compile repeats the choice
// without timing anything.
#ifndef FLUIDML_AMD_HOST_STRUCTURE_KERNEL_TUNER_H_
#define FLUIDML_AMD_HOST_STRUCTURE_KERNEL_TUNER_H_

#include <cstdint>
#include <functional>
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "fluidml_hip.h"
#include "utils/json.h"

namespace fluidml {
namespace kernel {

struct ContractPick {
  int tile = FL_TILE_RULE;  // enum fl_contract_tile
  int splits = 0;           // workgroups per tile along K; 0: the library's rule
  double ns = 0;            // measured duration of the pick (0: not measured)
  double rule_ns = 0;       // measured duration of the library's rule on the same problem
  // the bits of fl_contract_flags that name this configuration
  uint32_t Flags() const { return FL_CONTRACT_TILE(tile) | FL_CONTRACT_SPLITS(splits); }
  bool IsRule() const { return tile == FL_TILE_RULE && splits == 0; }
};

class ContractionTable {
 public:
  enum class Mode {
    Off,      // every contraction runs with the library's rule (environment FLUIDML_TUNE=0)
    Measure,  // unknown signatures are timed on the device (the default)
    Replay    // only what the table already holds is used; unknown signatures get the rule (FLUIDML_TUNE=<json file>)
  };
  explicit ContractionTable(Mode mode = Mode::Measure) : mode_(mode) {}
  // FLUIDML_TUNE: unset or 1 = Measure, 0 = Off, anything else = path of a JSON file written by an earlier
  // compile (the table is read from its "contraction_table" member, or from the document itself)
  static ContractionTable FromEnvironment();

  Mode GetMode() const { return mode_; }
  void SetMode(Mode mode) { mode_ = mode; }
  bool Find(const std::string &signature, ContractPick *pick) const;
  void Put(const std::string &signature, const ContractPick &pick);
  size_t Size() const { return picks_.size(); }
  const std::map<std::string, ContractPick> &GetPicks() const { return picks_; }

  // {"<signature>":{"tile":t,"splits":s,"ns":n,"rule_ns":r},...}, keys in lexicographic order
  std::string ToJson() const;
  // accepts that object, or a document that holds it under "contraction_table"; entries replace equal signatures
  void LoadJson(const json::Value &doc);
  void LoadJsonText(const std::string &text);

  // Every (tile, splits) a tuner tries besides the rule: all tiles x {rule's split, 1, 2, 3, 4, 6, 8, 12, 16}
  // (`full`), or the short list used where many problems are priced (the layout DP): every tile with the rule's
  // split plus the rule's tile with 1, 2, 4 and 8 splits.
  static std::vector<std::pair<int, int>> Candidates(bool full);

  // The fastest admissible configuration of one problem.  `launch(flags)` issues the problem once with the given
  // fl_contract_flags bits and returns the C ABI's code (FL_ERR_UNSUPPORTED: skipped); `elapsed_ns()` returns the
  // device time of the launch just issued.  The rule is replaced only by a configuration at least `margin`
  // (fraction) faster, so that two compiles of one graph do not flip between equals.
  static ContractPick Measure(const std::vector<std::pair<int, int>> &candidates,
                              const std::function<int(uint32_t)> &launch, const std::function<double()> &elapsed_ns,
                              int rounds, double margin);

  // Signature of a problem: `kind` (entry point family), operand views, number of grouped right operands and a
  // free-form tag for the epilogue ("b1c6s0": bias, chain steps, addends ...).
  static std::string Signature(const std::string &kind, const fl_tensor &lhs, const fl_tensor &rhs, const fl_tensor &out,
                               int group, const std::string &epilogue);

 private:
  Mode mode_;
  std::map<std::string, ContractPick> picks_;
};

// margin by which a configuration has to beat the rule to replace it
constexpr double kTuneMargin = 0.015;

}  // namespace kernel
}  // namespace fluidml

#endif
