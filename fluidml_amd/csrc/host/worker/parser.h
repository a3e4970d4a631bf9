// ONNX file -> graph::Graph (reference include/worker/parser.h, src/worker/parser.cpp).
#ifndef FLUIDML_AMD_HOST_WORKER_PARSER_H_
#define FLUIDML_AMD_HOST_WORKER_PARSER_H_

#include <istream>
#include <memory>
#include <string_view>

#include "structure/graph/graph.h"

namespace fluidml {
namespace worker {

class Parser {
 public:
  virtual ~Parser() = default;
  graph::Graph Run(std::string_view path);
  graph::Graph Run(std::istream &input);
  // serialized ModelProto bytes
  virtual graph::Graph RunOnBytes(const std::string &bytes) = 0;
  static std::unique_ptr<Parser> Make();
};

}  // namespace worker
}  // namespace fluidml

#endif
