// Runs the compiled plan on caller-owned host buffers (reference
// include/worker/runner.h, src/worker/runner.cpp:56-135).
#ifndef FLUIDML_AMD_HOST_WORKER_RUNNER_H_
#define FLUIDML_AMD_HOST_WORKER_RUNNER_H_

#include <memory>
#include <string>
#include <unordered_map>

#ifdef BUILD_PYTHON
#include "pybind11/numpy.h"
#endif

#include "structure/context/context.h"

namespace fluidml {
namespace worker {

class Runner {
 public:
  virtual ~Runner() = default;
  // `args` maps the ONNX value name of every graph input and output to a dense
  // row-major host buffer of exactly the tensor's size; outputs are written in
  // place.  Returns the mean wall-clock nanoseconds of one of the `epoch`
  // back-to-back replays.  Throws std::out_of_range when a name is missing
  // (reference runner.cpp:70) and std::runtime_error on a device error.
  virtual size_t Run(const std::unordered_map<std::string, void *> &args, size_t epoch = 1) = 0;
#ifdef BUILD_PYTHON
  // same, taking each array's buffer pointer; unlike the reference
  // (runner.cpp:123-135) the byte size of every array is checked
  virtual size_t Run(const std::unordered_map<std::string, pybind11::array> &args, size_t epoch = 1) = 0;
#endif
  static std::unique_ptr<Runner> Make(context::Context &&context);
};

}  // namespace worker
}  // namespace fluidml

#endif
