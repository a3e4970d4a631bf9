#include "worker/utils.h"

#include <stdexcept>

namespace fluidml {
namespace worker {

std::string GetBufferName(const std::string &name) { return name + "-buffer"; }

std::unique_ptr<kernel::Kernel> SelectKernel(const flow::Node *node) {
  if (node == nullptr) throw std::invalid_argument("SelectKernel: null node");
  return kernel::MakeKernel(node->GetKind(), node->GetAttrs());
}

std::unique_ptr<kernel::KernelGenerator> SelectKernelGenerator(const flow::Node *node) {
  if (node == nullptr) throw std::invalid_argument("SelectKernelGenerator: null node");
  return std::make_unique<kernel::KernelGenerator>(*node);
}

}  // namespace worker
}  // namespace fluidml
