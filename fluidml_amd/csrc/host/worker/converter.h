// graph::Graph -> flow::Flow (reference include/worker/converter.h,
// src/worker/converter.cpp): picks the operator variant from which inputs are
// constants and creates regions, nodes and def/use edges.
#ifndef FLUIDML_AMD_HOST_WORKER_CONVERTER_H_
#define FLUIDML_AMD_HOST_WORKER_CONVERTER_H_

#include <memory>

#include "structure/flow/flow.h"
#include "structure/graph/graph.h"

namespace fluidml {
namespace worker {

class Converter {
 public:
  virtual ~Converter() = default;
  // Throws std::runtime_error for an operand pattern the reference leaves
  // unreachable (it has no error path: DEBUG assert / release UB).
  virtual flow::Flow Run(const graph::Graph &graph) = 0;
  static std::unique_ptr<Converter> Make();
};

}  // namespace worker
}  // namespace fluidml

#endif
