// MaxPool / AveragePool without padding (HBM bound).
//
// The reference takes one strided subview of the input per kernel offset, in
// utils::GenAllIndicesInOrder order, and folds them with arith.maximumf
// (maxpool.cpp:17-82) or a left-to-right addf chain followed by one divf
// (averagepool.cpp:19-87).  One lane per output element walks the window in
// that same row-major order, so the average is bit-identical to the
// reference's addition order.
#include "fl_common.h"

namespace fl {
namespace {

constexpr int kBlock = 256;

struct PoolArgs {
  NestArgs<2> nest;    // operand 0 = out, 1 = in with spatial strides pre-multiplied by the pool stride
  NestArgs<1> window;  // kernel dims, input strides
  uint32_t n_out;
  uint32_t n_window;
};

__device__ __forceinline__ float MaximumF(float a, float b) {
  float r = fmaxf(a, b);
  if (a != a) r = a;
  if (b != b) r = b;
  return r;
}

template <bool IS_MAX>
__global__ __launch_bounds__(kBlock) void PoolKernel(PoolArgs p, float *__restrict__ out,
                                                     const float *__restrict__ in) {
  const uint32_t item = blockIdx.x * kBlock + threadIdx.x;
  if (item >= p.n_out) return;
  int32_t off[2] = {0, 0};
  p.nest.AddOffsets(item, off);
  const int32_t off0 = off[0];
  const float *src = in + off[1];
  float acc = src[0];
  for (uint32_t w = 1; w < p.n_window; ++w) {
    int32_t woff[1] = {0};
    p.window.AddOffsets(w, woff);
    const float v = src[woff[0]];
    acc = IS_MAX ? MaximumF(acc, v) : acc + v;
  }
  out[off0] = IS_MAX ? acc : acc / static_cast<float>(p.n_window);
}

template <bool IS_MAX>
int Pool(const fl_tensor *in, const fl_tensor *out, const int64_t *kernel_shape, const int64_t *strides, int32_t n,
         void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (in->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  if (in->rank != out->rank) return FL_ERR_RANK;
  if (n <= 0 || n > in->rank || kernel_shape == nullptr || strides == nullptr) return FL_ERR_ATTR;
  const int batches = in->rank - n;
  LoopNest nest, window;
  nest.rank = out->rank;
  nest.n_operands = 2;
  window.rank = n;
  window.n_operands = 1;
  int64_t n_window = 1;
  for (int i = 0; i < out->rank; ++i) {
    nest.shape[i] = out->shape[i];
    nest.strides[0][i] = out->strides[i];
    if (i < batches) {
      if (in->shape[i] != out->shape[i]) return FL_ERR_SHAPE;
      nest.strides[1][i] = in->strides[i];
    } else {
      const int k = i - batches;
      if (kernel_shape[k] <= 0 || strides[k] <= 0) return FL_ERR_ATTR;
      // the last window must lie inside the input
      if ((out->shape[i] - 1) * strides[k] + kernel_shape[k] > in->shape[i]) return FL_ERR_SHAPE;
      nest.strides[1][i] = in->strides[i] * strides[k];
      window.shape[k] = kernel_shape[k];
      window.strides[0][k] = in->strides[i];
      n_window *= kernel_shape[k];
    }
  }
  nest.Canonicalise();
  // the window keeps its logical (row-major) order: that is the fold order
  PoolArgs p;
  p.nest = MakeNestArgs<2>(nest);
  p.window = MakeNestArgs<1>(window);
  p.n_out = static_cast<uint32_t>(Numel(out));
  p.n_window = static_cast<uint32_t>(n_window);
  FL_LAUNCH(PoolKernel<IS_MAX>, dim3((p.n_out + kBlock - 1) / kBlock), dim3(kBlock), 0, AsStream(stream), p,
                     static_cast<float *>(out->base), static_cast<const float *>(in->base));
  return LaunchStatus();
}

}  // namespace
}  // namespace fl

extern "C" {

int fluidml_hip_max_pool_without_padding(const fl_tensor *in, const fl_tensor *out, const int64_t *kernel_shape,
                                         const int64_t *strides, int32_t n, void *stream) {
  return fl::Pool<true>(in, out, kernel_shape, strides, n, stream);
}

int fluidml_hip_average_pool_without_padding(const fl_tensor *in, const fl_tensor *out, const int64_t *kernel_shape,
                                             const int64_t *strides, int32_t n, void *stream) {
  return fl::Pool<false>(in, out, kernel_shape, strides, n, stream);
}

}  // extern "C"
