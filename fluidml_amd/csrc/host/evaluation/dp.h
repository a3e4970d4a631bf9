// Layout selection by dynamic programming over measured kernel costs
// (reference include/evaluation/dp.h, src/evaluation/dp.cpp).
#ifndef FLUIDML_AMD_HOST_EVALUATION_DP_H_
#define FLUIDML_AMD_HOST_EVALUATION_DP_H_

#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "structure/flow/flow.h"

namespace fluidml {
namespace worker {
class Evaluator;
}
namespace evaluation {

class CostModel;

// tensor name -> chosen layout (reference dp.h:13-40)
class DynamicProgrammingPlan {
 public:
  DynamicProgrammingPlan() = default;
  explicit DynamicProgrammingPlan(std::unordered_map<std::string, std::vector<size_t>> &&plan);
  DynamicProgrammingPlan(const DynamicProgrammingPlan &) = delete;
  DynamicProgrammingPlan(DynamicProgrammingPlan &&) = default;
  DynamicProgrammingPlan &operator=(DynamicProgrammingPlan &&) = default;
  bool HasLayout(const std::string &name) const;
  const std::vector<size_t> &GetLayout(const std::string &name) const;
  const std::unordered_map<std::string, std::vector<size_t>> &GetAll() const { return plan_; }
  // {"tensor": [layout...], ...}, keys sorted (reference dp.cpp:877-884)
  std::string ToJson() const;
  // union; on a name both hold, `lhs` wins (reference dp.cpp:861-875)
  friend DynamicProgrammingPlan Merge(const DynamicProgrammingPlan &lhs, const DynamicProgrammingPlan &rhs);

 private:
  std::unordered_map<std::string, std::vector<size_t>> plan_;
};

DynamicProgrammingPlan Merge(const DynamicProgrammingPlan &lhs, const DynamicProgrammingPlan &rhs);

class DynamicProgrammingTable {
 public:
  virtual ~DynamicProgrammingTable() = default;
  virtual DynamicProgrammingPlan Run(const flow::Flow &flow) = 0;
  // {"evaluator": {<KernelName>: [{"shapes":…, "layouts":…, "time_cost":…}…]}} (reference
  // evaluator.cpp:123-138, eval.cpp:136-152)
  virtual std::string ToJson() const = 0;
  // `cost` answers "how long does this kernel take with these layouts"
  static std::unique_ptr<DynamicProgrammingTable> Make(std::shared_ptr<CostModel> cost);
};

}  // namespace evaluation
}  // namespace fluidml

#endif
