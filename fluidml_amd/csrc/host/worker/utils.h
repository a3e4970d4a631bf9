// Node -> kernel dispatch (reference include/worker/utils.h:13-16,
// src/worker/utils.cpp:80-335 SelectKernel, :337-966 SelectKernelGenerator).
#ifndef FLUIDML_AMD_HOST_WORKER_UTILS_H_
#define FLUIDML_AMD_HOST_WORKER_UTILS_H_

#include <memory>
#include <string>

#include "structure/flow/flow.h"
#include "structure/kernel/generator.h"
#include "structure/kernel/kernel.h"

namespace fluidml {
namespace worker {

// symbol under which a node's scratch is known (reference utils.cpp:76-78)
std::string GetBufferName(const std::string &name);
std::unique_ptr<kernel::Kernel> SelectKernel(const flow::Node *node);
std::unique_ptr<kernel::KernelGenerator> SelectKernelGenerator(const flow::Node *node);

}  // namespace worker
}  // namespace fluidml

#endif
