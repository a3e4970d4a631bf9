// Compile-then-run entry point (reference include/worker/executor.h:15-45,
// src/worker/executor.cpp).
#ifndef FLUIDML_AMD_HOST_WORKER_EXECUTOR_H_
#define FLUIDML_AMD_HOST_WORKER_EXECUTOR_H_

#include <fstream>
#include <istream>
#include <memory>
#include <optional>
#include <string>
#include <string_view>
#include <unordered_map>

#ifdef BUILD_PYTHON
#include "pybind11/numpy.h"
#endif

#include "structure/context/context.h"

namespace fluidml {
namespace worker {

class Executor {
 public:
  virtual ~Executor() = default;
  // Parser -> Converter -> Planner -> GeneralBuilder -> Lower, in that order
  // (reference executor.cpp:91-114).  `mlir` and `llvm` receive the textual
  // launch plan (there is no IR to dump), `json` the layout-DP report.
  virtual void Compile(std::istream &input, std::ofstream *mlir = nullptr, std::ofstream *llvm = nullptr,
                       std::ofstream *json = nullptr) = 0;
  virtual void Compile(std::string_view input, std::optional<std::string_view> mlir = std::nullopt,
                       std::optional<std::string_view> llvm = std::nullopt,
                       std::optional<std::string_view> json = std::nullopt) = 0;
  // mean nanoseconds per epoch (reference executor.cpp:135-139)
  virtual size_t Invoke(const std::unordered_map<std::string, void *> &args) = 0;
#ifdef BUILD_PYTHON
  virtual size_t Invoke(const std::unordered_map<std::string, pybind11::array> &args) = 0;
#endif
  // the shared compilation state (launch plan, options); not in the reference's interface
  virtual context::Context &GetContext() = 0;

  static std::unique_ptr<Executor> MakePlainLinear(std::string &&name, size_t epoch = 1);
  static std::unique_ptr<Executor> MakePlainGreedy(std::string &&name, size_t epoch = 1);
  static std::unique_ptr<Executor> MakeDPGreedy(std::string &&name, size_t epoch = 1);

 protected:
  Executor() = default;
  Executor(const Executor &) = delete;
  Executor(Executor &&) = default;
};

}  // namespace worker
}  // namespace fluidml

#endif
