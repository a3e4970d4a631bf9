// Kernels of the hot path as launchable objects.
//
// The reference's kernel classes emit MLIR through `Run(mlir::OpBuilder&,
// mlir::Value&...)` (include/structure/kernel/kernel/kernel.h:40-88).  Here the
// same four families launch gfx950 kernels through the C ABI of
// include/fluidml_hip.h: `mlir::OpBuilder&` becomes a LaunchContext (stream +
// literal-reference flags + first error), `mlir::Value&` becomes a TensorView
// (device pointer, element type, shape, element strides -- what the reference
// kernels read from the memref type), and the i8 scratch memref becomes a
// Buffer.  GetKernelName() returns the reference's kKernelName strings, which
// are also the keys of the layout-DP cost table.
#ifndef FLUIDML_AMD_HOST_STRUCTURE_KERNEL_KERNEL_H_
#define FLUIDML_AMD_HOST_STRUCTURE_KERNEL_KERNEL_H_

#include <memory>
#include <string>
#include <vector>

#include "fluidml_hip.h"
#include "structure/flow/flow.h"
#include "structure/tensor/meta.h"
#include "structure/tensor/tensor.h"

namespace fluidml {
namespace kernel {

// the six loop orders the reference autotunes MatMul/Gemm over (kernel/utils.h:12-14,
// utils.cpp:9-13); kept as the key space of the autotune cache
enum Axis { i = 0, j = 1, k = 2 };
std::vector<std::vector<Axis>> GetAxesInAllOrders();

struct LaunchContext {
  void *stream = nullptr;  // hipStream_t
  uint32_t flags = 0;      // FL_REF_* literal-reference switches
  bool bf16 = false;       // MatMul on the opt-in bf16 path (operands rounded to bf16, fp32 accumulation)
  // tile configuration and K splits for the contraction about to be launched (FL_CONTRACT_TILE / FL_CONTRACT_SPLITS
  // bits); 0: the kernel object's own choice, and failing that the library's rule
  uint32_t contract = 0;
  int status = 0;          // first non-zero return code of the C ABI
  std::string failed;      // kernel name that produced it
  void Note(int code, const std::string &kernel_name);
};

struct TensorView {
  fl_tensor t;
  TensorView();
  // `base` points at logical element 0; strides follow from shape + layout
  TensorView(void *base, const Meta &meta, const std::vector<size_t> &layout);
  TensorView(void *base, const Meta &meta);  // identity layout
};

struct Buffer {
  void *ptr = nullptr;
  size_t bytes = 0;
};

// A constant a kernel owns (bias, scale, gather table, where-condition, ...):
// kept on the host until Upload() copies it to HBM once.
class DeviceConstant {
 public:
  explicit DeviceConstant(const Tensor &tensor);
  ~DeviceConstant();
  DeviceConstant(const DeviceConstant &) = delete;
  void Upload();  // idempotent; throws std::runtime_error on a HIP error
  bool IsUploaded() const { return device_ != nullptr; }
  TensorView View() const;  // valid after Upload()
  size_t GetSize() const { return tensor_.GetMeta().GetSize(); }

 private:
  Tensor tensor_;
  void *device_ = nullptr;
};

class Kernel {
 public:
  virtual ~Kernel() = default;
  virtual std::string GetKernelName() const = 0;
  // copies the kernel's own constants to HBM (no-op for most kernels); must run
  // before the first Run and outside any stream capture
  virtual void Prepare() {}
  // bytes of HBM the kernel's own constants occupy
  virtual size_t GetConstantBytes() const { return 0; }
  // i-th constant the kernel owns (0..2), nullptr if it has none there; lets a fused launch reuse
  // the uploaded LayerNorm scale/bias of the node it absorbs
  virtual const DeviceConstant *GetConstant(int i) const {
    (void)i;
    return nullptr;
  }
  // MatMul / Gemm: the tile configuration this kernel object launches with (FL_CONTRACT_TILE / FL_CONTRACT_SPLITS
  // bits, 0 = the library's rule) -- what the reference's generator fixes by picking one of its loop orders
  // (generator/matmul.cpp:88-131).  Ignored by every other kernel.
  virtual void SetContractFlags(uint32_t bits) { (void)bits; }
  virtual uint32_t GetContractFlags() const { return 0; }
};

class SingleInputKernel : virtual public Kernel {};
class DoubleInputsKernel : virtual public Kernel {};

class SingleInputWithoutBufferKernel : public SingleInputKernel {
 public:
  virtual void Run(LaunchContext &ctx, const TensorView &input, const TensorView &output) const = 0;
};

class SingleInputWithBufferKernel : public SingleInputKernel {
 public:
  virtual void Run(LaunchContext &ctx, const TensorView &input, const TensorView &output, const Buffer &buffer) const = 0;
};

class DoubleInputsWithoutBufferKernel : public DoubleInputsKernel {
 public:
  virtual void Run(LaunchContext &ctx, const TensorView &lhs, const TensorView &rhs, const TensorView &output) const = 0;
};

class DoubleInputsWithBufferKernel : public DoubleInputsKernel {
 public:
  virtual void Run(LaunchContext &ctx, const TensorView &lhs, const TensorView &rhs, const TensorView &output,
                   const Buffer &buffer) const = 0;
};

// kKernelName of the reference class that serves `kind` (note
// GemmConstantWeightsBias -> "GemmConstantWeightsBiasKernel", reference gemm.h:13).
std::string KernelNameOf(flow::OpKind kind);

// The concrete kernel for a node kind and its attributes; the returned object
// belongs to exactly one of the four families above, the one
// flow::Node::IsSingleInput()/HasBuffer() name.
std::unique_ptr<Kernel> MakeKernel(flow::OpKind kind, const flow::Attrs &attrs);

}  // namespace kernel
}  // namespace fluidml

#endif
