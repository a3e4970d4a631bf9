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

// 2x2 window, stride 2, unit-stride rows on both sides (the pools of the VGG/ResNet families): a lane reads
// 2*OUTS consecutive values of two input rows with 128-bit loads and writes OUTS consecutive outputs.  The
// window is folded in its row-major order like PoolKernel does, so the results are identical.
template <bool IS_MAX, int OUTS>
__global__ __launch_bounds__(kBlock) void Pool2x2Kernel(NestArgs<2> nest, uint32_t n_items, int32_t row_stride,
                                                        bool streaming, float *__restrict__ out,
                                                        const float *__restrict__ in) {
  const uint32_t item = blockIdx.x * kBlock + threadIdx.x;
  if (item >= n_items) return;
  int32_t off[2] = {0, 0};
  nest.AddOffsets(item, off);
  const float *src = in + off[1];
  struct alignas(16) Quad {
    float v[4];
  };
  struct alignas(4 * OUTS) Outs {
    float v[OUTS];
  };
  float top[2 * OUTS], bottom[2 * OUTS];
#pragma unroll
  for (int q = 0; q < OUTS / 2; ++q) {
    const Quad t = reinterpret_cast<const Quad *>(src)[q], b = reinterpret_cast<const Quad *>(src + row_stride)[q];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      top[4 * q + k] = t.v[k];
      bottom[4 * q + k] = b.v[k];
    }
  }
  Outs r;
#pragma unroll
  for (int k = 0; k < OUTS; ++k) {
    float acc = top[2 * k];
    acc = IS_MAX ? MaximumF(acc, top[2 * k + 1]) : acc + top[2 * k + 1];
    acc = IS_MAX ? MaximumF(acc, bottom[2 * k]) : acc + bottom[2 * k];
    acc = IS_MAX ? MaximumF(acc, bottom[2 * k + 1]) : acc + bottom[2 * k + 1];
    r.v[k] = IS_MAX ? acc : acc / 4.0f;
  }
  StoreMaybeStreaming(reinterpret_cast<Outs *>(out + off[0]), r, streaming);
}

// Launches Pool2x2Kernel when the canonical nest allows it; false = use the generic kernel.
template <bool IS_MAX>
bool TryPool2x2(LoopNest nest, const LoopNest &window, const fl_tensor *in, const fl_tensor *out, hipStream_t stream) {
  if (window.rank != 2 || window.shape[0] != 2 || window.shape[1] != 2 || window.strides[0][1] != 1) return false;
  const int inner = nest.rank - 1;
  if (inner < 0 || nest.strides[0][inner] != 1 || nest.strides[1][inner] != 2) return false;
  const int64_t row_stride = window.strides[0][0];
  const int outs = nest.shape[inner] % 4 == 0 ? 4 : nest.shape[inner] % 2 == 0 ? 2 : 0;
  if (outs == 0 || row_stride % 4 != 0 || row_stride > INT32_MAX) return false;
  if (!IsAligned(in->base, 16) || !IsAligned(out->base, 4 * outs)) return false;
  for (int d = 0; d < inner; ++d) {
    if (nest.strides[1][d] % 4 != 0 || nest.strides[0][d] % outs != 0) return false;
  }
  const int64_t n_out = Numel(out);
  nest.shape[inner] /= outs;
  nest.strides[0][inner] = outs;
  nest.strides[1][inner] = 2 * outs;
  const uint32_t n_items = static_cast<uint32_t>(n_out / outs);
  const NestArgs<2> args = MakeNestArgs<2>(nest);
  const bool streaming = StreamingOutput(static_cast<size_t>(n_out) * sizeof(float));
  const dim3 grid((n_items + kBlock - 1) / kBlock);
  if (outs == 4) {
    FL_LAUNCH((Pool2x2Kernel<IS_MAX, 4>), grid, dim3(kBlock), 0, stream, args, n_items, static_cast<int32_t>(row_stride),
              streaming, static_cast<float *>(out->base), static_cast<const float *>(in->base));
  } else {
    FL_LAUNCH((Pool2x2Kernel<IS_MAX, 2>), grid, dim3(kBlock), 0, stream, args, n_items, static_cast<int32_t>(row_stride),
              streaming, static_cast<float *>(out->base), static_cast<const float *>(in->base));
  }
  return true;
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
  if (Numel(out) <= INT32_MAX && TryPool2x2<IS_MAX>(nest, window, in, out, AsStream(stream))) return LaunchStatus();
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
