// Row-reduction kernels (HBM bound): Softmax, LayerNormalization, ReduceMean.
//
// The reference runs these as chains of linalg.generic passes over a scratch
// tensor (softmax.cpp:22-139 six passes, layer_normalization.cpp:33-220 seven,
// reduce_mean.cpp:16-98 three).  Here a row is read once, reduced in
// registers with wave64 shuffles (LDS only to combine waves) and written once.
//
// Two traversal shapes cover every layout the planner can pick:
//   * "row"    - the reduced axis is contiguous for input and output: one wave
//                (or one block) per row, lanes stride the row;
//   * "column" - the axis is strided: one lane per row, rows enumerated in the
//                output's physical order so neighbouring lanes touch
//                neighbouring addresses while each walks its axis.
#include "fl_common.h"

namespace fl {
namespace {

constexpr int kBlock = 256;

template <int NOPS>
struct RowArgs {
  uint32_t n_rows;
  uint32_t len;
  uint32_t streaming;  // 1 = the output is large enough for non-temporal stores
  int32_t axis_stride[NOPS];
  NestArgs<NOPS> outer;  // non-axis dims, canonical order (operand 0 = output)
};

template <int NOPS>
__device__ __forceinline__ void RowOffsets(const NestArgs<NOPS> &a, uint32_t row, int32_t *off) {
  int32_t acc[NOPS];
#pragma unroll
  for (int o = 0; o < NOPS; ++o) acc[o] = 0;
  a.AddOffsets(row, acc);
#pragma unroll
  for (int o = 0; o < NOPS; ++o) off[o] = acc[o];
}

// Build the outer nest (all dims but `axis`) for the given operands' strides.
template <int NOPS>
RowArgs<NOPS> MakeRowArgs(int rank, const int64_t *shape, int axis, const int64_t (*strides)[kMaxRank]) {
  static_assert(NOPS <= kMaxOperands, "LoopNest holds strides for kMaxOperands operands");
  LoopNest nest;
  nest.n_operands = NOPS;
  nest.rank = 0;
  for (int i = 0; i < rank; ++i) {
    if (i == axis) continue;
    nest.shape[nest.rank] = shape[i];
    for (int o = 0; o < NOPS; ++o) nest.strides[o][nest.rank] = strides[o][i];
    ++nest.rank;
  }
  nest.Canonicalise();
  RowArgs<NOPS> args;
  args.outer = MakeNestArgs<NOPS>(nest);
  int64_t rows = 1;
  for (int i = 0; i < nest.rank; ++i) rows *= nest.shape[i];
  args.n_rows = static_cast<uint32_t>(rows);
  args.len = static_cast<uint32_t>(shape[axis]);
  args.streaming = StreamingOutput(static_cast<size_t>(rows) * static_cast<size_t>(shape[axis]) * sizeof(float)) ? 1 : 0;
  for (int o = 0; o < NOPS; ++o) args.axis_stride[o] = static_cast<int32_t>(strides[o][axis]);
  return args;
}

// True when operand `o` of a row kernel can be read or written 16 bytes at a time along the axis: unit axis
// stride, every row starting on a 16-byte boundary.
inline bool RowsVectorisable(const void *base, int rank, const int64_t *shape, int axis, const int64_t *strides) {
  if (!IsAligned(base, 16) || (shape[axis] > 1 && strides[axis] != 1)) return false;
  for (int i = 0; i < rank; ++i) {
    if (i != axis && shape[i] > 1 && strides[i] % 4 != 0) return false;
  }
  return true;
}
// True when an operand's address depends only on the position along the axis (scale and bias of a
// LayerNormalization over the last dim).
inline bool RowInvariant(int rank, const int64_t *shape, int axis, const int64_t *strides) {
  for (int i = 0; i < rank; ++i) {
    if (i != axis && shape[i] > 1 && strides[i] != 0) return false;
  }
  return true;
}
// Row kernels switch to the many-rows variants from this many elements on (below, the launches of the
// transformer graphs keep the kernels they were tuned with).
constexpr int64_t kManyRowsElements = int64_t{1} << 20;

// ---- Softmax ----------------------------------------------------------------

// One wave per row, row cached in registers: len <= 64 * ITEMS.
// Optional prologue shared by the softmax kernels: x / div + mask (operand 2 of the nest, broadcast
// strides), i.e. the DivConstantRhs -> AddCommon -> Softmax chain of an attention block in one pass.
struct SoftmaxPre {
  const float *mask;  // nullptr = plain softmax
  float div;
  __device__ __forceinline__ float operator()(float x, int32_t mask_off) const {
    return mask != nullptr ? x / div + mask[mask_off] : x;
  }
};

template <int ITEMS>
__global__ __launch_bounds__(kBlock) void SoftmaxRowWave(RowArgs<3> a, float *__restrict__ out,
                                                         const float *__restrict__ in, SoftmaxPre pre) {
  const uint32_t lane = threadIdx.x % kWave;
  const uint32_t row = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (row >= a.n_rows) return;
  int32_t off[3];
  RowOffsets<3>(a.outer, row, off);
  const float *src = in + off[1];
  float *dst = out + off[0];
  const int32_t sm = a.axis_stride[2];
  float x[ITEMS];
  float m = -__FLT_MAX__;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = lane + i * kWave;
    x[i] = j < a.len ? pre(src[j], off[2] + static_cast<int32_t>(j) * sm) : -__FLT_MAX__;
    m = fmaxf(m, x[i]);
  }
  m = WaveReduce(m, MaxOp{});
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = lane + i * kWave;
    x[i] = j < a.len ? expf(x[i] - m) : 0.0f;
    s += x[i];
  }
  s = WaveReduce(s, SumOp{});
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = lane + i * kWave;
    if (j < a.len) StoreMaybeStreaming(dst + j, x[i] / s, a.streaming != 0);
  }
}

// Many short rows: LANES lanes per row (64 / LANES rows per wave), 128-bit accesses, row cached in registers:
// len <= 4 * LANES * ITEMS, len % 4 == 0, rows 16-byte aligned on both sides.
struct alignas(16) Quad {
  float v[4];
};

template <int LANES, typename F>
__device__ __forceinline__ float GroupReduce(float v, F f) {
#pragma unroll
  for (int off = LANES / 2; off > 0; off >>= 1) v = f(v, __shfl_xor(v, off, kWave));
  return v;
}

template <int LANES, int ITEMS>
__global__ __launch_bounds__(kBlock) void SoftmaxRowVec(RowArgs<3> a, float *__restrict__ out,
                                                        const float *__restrict__ in, SoftmaxPre pre) {
  const uint32_t lane = threadIdx.x % LANES;
  const uint32_t row = blockIdx.x * (kBlock / LANES) + threadIdx.x / LANES;
  if (row >= a.n_rows) return;  // a row's lanes leave together
  int32_t off[3];
  RowOffsets<3>(a.outer, row, off);
  const Quad *src = reinterpret_cast<const Quad *>(in + off[1]);
  Quad *dst = reinterpret_cast<Quad *>(out + off[0]);
  const int32_t sm = a.axis_stride[2];
  const uint32_t n_quads = a.len / 4;
  Quad x[ITEMS];
  float m = -__FLT_MAX__;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t q = lane + i * LANES;
    if (q < n_quads) x[i] = src[q];
  }
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t q = lane + i * LANES;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      x[i].v[k] = q < n_quads ? pre(x[i].v[k], off[2] + static_cast<int32_t>(4 * q + k) * sm) : -__FLT_MAX__;
      m = fmaxf(m, x[i].v[k]);
    }
  }
  m = GroupReduce<LANES>(m, MaxOp{});
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t q = lane + i * LANES;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      x[i].v[k] = q < n_quads ? expf(x[i].v[k] - m) : 0.0f;
      s += x[i].v[k];
    }
  }
  s = GroupReduce<LANES>(s, SumOp{});
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t q = lane + i * LANES;
    if (q < n_quads) {
      Quad r;
#pragma unroll
      for (int k = 0; k < 4; ++k) r.v[k] = x[i].v[k] / s;
      StoreMaybeStreaming(dst + q, r, a.streaming != 0);
    }
  }
}

// One block per row, any length, three passes over the (cache-resident) row.
__global__ __launch_bounds__(kBlock) void SoftmaxRowBlock(RowArgs<3> a, float *__restrict__ out,
                                                          const float *__restrict__ in, SoftmaxPre pre) {
  __shared__ float smem[kBlock / kWave];
  int32_t off[3];
  RowOffsets<3>(a.outer, blockIdx.x, off);
  const float *src = in + off[1];
  float *dst = out + off[0];
  const int32_t sm = a.axis_stride[2];
  auto at = [&](uint32_t j) { return pre(src[j], off[2] + static_cast<int32_t>(j) * sm); };
  float m = -__FLT_MAX__;
  for (uint32_t j = threadIdx.x; j < a.len; j += kBlock) m = fmaxf(m, at(j));
  m = BlockReduce<kBlock / kWave>(m, MaxOp{}, smem);
  float s = 0.0f;
  for (uint32_t j = threadIdx.x; j < a.len; j += kBlock) s += expf(at(j) - m);
  s = BlockReduce<kBlock / kWave>(s, SumOp{}, smem);
  for (uint32_t j = threadIdx.x; j < a.len; j += kBlock) dst[j] = expf(at(j) - m) / s;
}

// One block per row, row cached in registers: len <= 256 * ITEMS (read once, written once).
template <int ITEMS>
__global__ __launch_bounds__(kBlock) void SoftmaxRowBlockCached(RowArgs<3> a, float *__restrict__ out,
                                                                const float *__restrict__ in, SoftmaxPre pre) {
  __shared__ float smem[kBlock / kWave];
  int32_t off[3];
  RowOffsets<3>(a.outer, blockIdx.x, off);
  const float *src = in + off[1];
  float *dst = out + off[0];
  const int32_t sm = a.axis_stride[2];
  float x[ITEMS];
  float m = -__FLT_MAX__;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = threadIdx.x + i * kBlock;
    x[i] = j < a.len ? pre(src[j], off[2] + static_cast<int32_t>(j) * sm) : -__FLT_MAX__;
    m = fmaxf(m, x[i]);
  }
  m = BlockReduce<kBlock / kWave>(m, MaxOp{}, smem);
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = threadIdx.x + i * kBlock;
    x[i] = j < a.len ? expf(x[i] - m) : 0.0f;
    s += x[i];
  }
  s = BlockReduce<kBlock / kWave>(s, SumOp{}, smem);
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = threadIdx.x + i * kBlock;
    if (j < a.len) StoreMaybeStreaming(dst + j, x[i] / s, a.streaming != 0);
  }
}

// One lane per row; the axis is walked with its stride.
__global__ __launch_bounds__(kBlock) void SoftmaxColumn(RowArgs<3> a, float *__restrict__ out,
                                                        const float *__restrict__ in, SoftmaxPre pre) {
  const uint32_t row = blockIdx.x * kBlock + threadIdx.x;
  if (row >= a.n_rows) return;
  int32_t off[3];
  RowOffsets<3>(a.outer, row, off);
  const float *src = in + off[1];
  float *dst = out + off[0];
  const int32_t si = a.axis_stride[1], so = a.axis_stride[0], sm = a.axis_stride[2];
  auto at = [&](uint32_t j) { return pre(src[static_cast<int32_t>(j) * si], off[2] + static_cast<int32_t>(j) * sm); };
  float m = -__FLT_MAX__;
  for (uint32_t j = 0; j < a.len; ++j) m = fmaxf(m, at(j));
  float s = 0.0f;
  for (uint32_t j = 0; j < a.len; ++j) s += expf(at(j) - m);
  for (uint32_t j = 0; j < a.len; ++j) dst[static_cast<int32_t>(j) * so] = expf(at(j) - m) / s;
}

// ---- LayerNormalization -------------------------------------------------------

// operands: 0 out, 1 in, 2 scale, 3 bias, 4 scratch (one float per row), 5 optional addend y: LN(in + y)
template <int ITEMS>
__global__ __launch_bounds__(kBlock) void LayerNormRowBlock(RowArgs<6> a, float *__restrict__ out,
                                                            const float *__restrict__ in,
                                                            const float *__restrict__ scale,
                                                            const float *__restrict__ bias,
                                                            const float *__restrict__ scratch, float eps,
                                                            int stale_scratch, const float *__restrict__ addend) {
  __shared__ float smem[kBlock / kWave];
  int32_t off[6];
  RowOffsets<6>(a.outer, blockIdx.x, off);
  const float *src = in + off[1];
  const float n = static_cast<float>(a.len);
  float x[ITEMS];
  float s = 0.0f;
  // scale and bias are requested together with the row: asked for after the two reductions they would be one more
  // memory round trip at the end of a kernel that is nothing but a chain of round trips
  const float *g = scale + off[2];
  const float *b = bias + off[3];
  const int32_t sg = a.axis_stride[2], sb = a.axis_stride[3];
  float gv[ITEMS], bv[ITEMS];
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = threadIdx.x + i * kBlock;
    x[i] = j < a.len ? src[j] : 0.0f;
    if (addend != nullptr && j < a.len) x[i] = x[i] + addend[off[5] + static_cast<int32_t>(j) * a.axis_stride[5]];
    gv[i] = j < a.len ? g[static_cast<int32_t>(j) * sg] : 0.0f;
    bv[i] = j < a.len ? b[static_cast<int32_t>(j) * sb] : 0.0f;
    s += x[i];
  }
  s = BlockReduce<kBlock / kWave>(s, SumOp{}, smem);
  if (stale_scratch) s += scratch[off[4]];
  const float mean = s / n;
  float v = 0.0f;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = threadIdx.x + i * kBlock;
    x[i] = j < a.len ? x[i] - mean : 0.0f;
    v += x[i] * x[i];
  }
  v = BlockReduce<kBlock / kWave>(v, SumOp{}, smem);
  const float inv = 1.0f / sqrtf(v / n + eps);
  float *dst = out + off[0];
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = threadIdx.x + i * kBlock;
    if (j < a.len) StoreMaybeStreaming(dst + j, (x[i] * inv) * gv[i] + bv[i], a.streaming != 0);
  }
}

// An embedding lookup, the embeddings added to it and the LayerNormalization behind them, one workgroup per looked-up
// row (len <= ITEMS * kBlock, every operand dense along the row):
//   v = (data0[idx0[row]] + second) + third,   second = data1[idx1[row]] or a tensor's row,   out = LN(v)
// The sums round like the separate Gather / AddCommon kernels; the statistics are the two passes of LayerNormRowBlock.
struct EmbedArgs {
  uint32_t len;
  int64_t rows0, rows1;          // rows of the tables (rows1 unused without idx1)
  uint32_t second_rows, third_rows;  // a tensor addend repeats after this many rows (leading dims of extent 1)
};
__device__ inline int64_t TableRow(int64_t idx, int64_t rows) {
  if (idx < 0) idx += rows;  // ONNX negative indexing
  return idx < 0 ? 0 : (idx >= rows ? rows - 1 : idx);  // never read outside the table
}
template <int ITEMS>
__global__ __launch_bounds__(kBlock) void EmbeddingLayerNormKernel(EmbedArgs a, float *__restrict__ out,
                                                                   const int64_t *__restrict__ idx0,
                                                                   const float *__restrict__ data0,
                                                                   const int64_t *__restrict__ idx1,
                                                                   const float *__restrict__ second,
                                                                   const float *__restrict__ third,
                                                                   const float *__restrict__ scale,
                                                                   const float *__restrict__ bias, float eps) {
  __shared__ float smem[kBlock / kWave];
  const uint32_t row = blockIdx.x;
  const float *r0 = data0 + TableRow(idx0[row], a.rows0) * a.len;
  const float *r1 = idx1 != nullptr ? second + TableRow(idx1[row], a.rows1) * a.len
                                    : second + static_cast<size_t>(row % a.second_rows) * a.len;
  const float *r2 = third != nullptr ? third + static_cast<size_t>(row % a.third_rows) * a.len : nullptr;
  const float n = static_cast<float>(a.len);
  float x[ITEMS], gv[ITEMS], bv[ITEMS];
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = threadIdx.x + i * kBlock;
    const bool in = j < a.len;
    x[i] = in ? r0[j] + r1[j] : 0.0f;
    if (r2 != nullptr && in) x[i] = x[i] + r2[j];
    gv[i] = in ? scale[j] : 0.0f;
    bv[i] = in ? bias[j] : 0.0f;
    s += x[i];
  }
  s = BlockReduce<kBlock / kWave>(s, SumOp{}, smem);
  const float mean = s / n;
  float v = 0.0f;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = threadIdx.x + i * kBlock;
    x[i] = j < a.len ? x[i] - mean : 0.0f;
    v += x[i] * x[i];
  }
  v = BlockReduce<kBlock / kWave>(v, SumOp{}, smem);
  const float inv = 1.0f / sqrtf(v / n + eps);
  float *dst = out + static_cast<size_t>(row) * a.len;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = threadIdx.x + i * kBlock;
    if (j < a.len) dst[j] = (x[i] * inv) * gv[i] + bv[i];
  }
}

// An embedding lookup that also leaves what a deferred LayerNormalization of its result needs: one workgroup per
// looked-up row copies the table row and writes (mean, sum of squared deviations) of every run of 32 columns,
// stats[(row * parts + run) * 2 + {0, 1}] -- the partial row statistics a contraction leaves with FL_NORM stats_out.
__global__ __launch_bounds__(kBlock) void GatherStatsKernel(uint32_t len, int64_t table_rows, float *__restrict__ out,
                                                            const int64_t *__restrict__ idx,
                                                            const float *__restrict__ data, float *__restrict__ stats) {
  const uint32_t row = blockIdx.x;
  const float *src = data + TableRow(idx[row], table_rows) * len;
  float *dst = out + static_cast<size_t>(row) * len;
  const uint32_t parts = (len + 31) / 32;
  for (uint32_t base = 0; base < len; base += kBlock) {  // (uniform trip count: the shuffles below need every lane)
    const uint32_t j = base + threadIdx.x;
    const bool in = j < len;
    const float x = in ? src[j] : 0.0f;
    if (in) dst[j] = x;
    const uint32_t first = j & ~31u;
    const float cols = static_cast<float>(first < len ? min(32u, len - first) : 1u);
    float sum = x;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    const float mean = sum / cols;
    const float d = in ? x - mean : 0.0f;
    float sq = d * d;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 64);
    if ((threadIdx.x & 31u) == 0 && in) {
      float *at = stats + (static_cast<size_t>(row) * parts + j / 32) * 2;
      at[0] = mean;
      at[1] = sq;
    }
  }
}

// One wave per row, row cached in registers: len <= 64 * ITEMS; no workgroup barrier at all.
template <int ITEMS>
__global__ __launch_bounds__(kBlock) void LayerNormRowWave(RowArgs<6> a, float *__restrict__ out,
                                                           const float *__restrict__ in,
                                                           const float *__restrict__ scale,
                                                           const float *__restrict__ bias,
                                                           const float *__restrict__ scratch, float eps,
                                                           int stale_scratch, const float *__restrict__ addend) {
  const uint32_t lane = threadIdx.x % kWave;
  const uint32_t row = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (row >= a.n_rows) return;
  int32_t off[6];
  RowOffsets<6>(a.outer, row, off);
  const float *src = in + off[1];
  const float n = static_cast<float>(a.len);
  float x[ITEMS];
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = lane + i * kWave;
    x[i] = j < a.len ? src[j] : 0.0f;
    if (addend != nullptr && j < a.len) x[i] = x[i] + addend[off[5] + static_cast<int32_t>(j) * a.axis_stride[5]];
    s += x[i];
  }
  s = WaveReduce(s, SumOp{});
  if (stale_scratch) s += scratch[off[4]];
  const float mean = s / n;
  float v = 0.0f;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = lane + i * kWave;
    x[i] = j < a.len ? x[i] - mean : 0.0f;
    v += x[i] * x[i];
  }
  v = WaveReduce(v, SumOp{});
  const float inv = 1.0f / sqrtf(v / n + eps);
  float *dst = out + off[0];
  const float *g = scale + off[2];
  const float *b = bias + off[3];
  const int32_t sg = a.axis_stride[2], sb = a.axis_stride[3];
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t j = lane + i * kWave;
    if (j < a.len) {
      StoreMaybeStreaming(dst + j, (x[i] * inv) * g[static_cast<int32_t>(j) * sg] + b[static_cast<int32_t>(j) * sb],
                          a.streaming != 0);
    }
  }
}

// Many rows: a workgroup copies scale and bias into LDS once, then each of its waves walks rows (one wave per
// row, 128-bit accesses, row cached in registers): len <= 256 * ITEMS, len % 4 == 0, rows (and the addend's)
// 16-byte aligned.  Dynamic LDS: 2 * len floats.
template <int ITEMS>
__global__ __launch_bounds__(kBlock) void LayerNormRowVec(RowArgs<6> a, float *__restrict__ out,
                                                          const float *__restrict__ in,
                                                          const float *__restrict__ scale,
                                                          const float *__restrict__ bias,
                                                          const float *__restrict__ scratch, float eps,
                                                          int stale_scratch, const float *__restrict__ addend) {
  extern __shared__ __align__(16) float ln_params[];  // scale[len], bias[len]
  const uint32_t lane = threadIdx.x % kWave;
  const uint32_t n_quads = a.len / 4;
  {
    // scale and bias do not depend on the row in this variant (the host checks it)
    const int32_t sg = a.axis_stride[2], sb = a.axis_stride[3];
    for (uint32_t j = threadIdx.x; j < a.len; j += kBlock) {
      ln_params[j] = scale[static_cast<int32_t>(j) * sg];
      ln_params[a.len + j] = bias[static_cast<int32_t>(j) * sb];
    }
  }
  __syncthreads();
  const Quad *gq = reinterpret_cast<const Quad *>(ln_params);
  const Quad *bq = reinterpret_cast<const Quad *>(ln_params + a.len);
  const float n = static_cast<float>(a.len);
  const uint32_t row_step = gridDim.x * (kBlock / kWave);
  for (uint32_t row = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave; row < a.n_rows; row += row_step) {
    int32_t off[6];
    RowOffsets<6>(a.outer, row, off);
    const Quad *src = reinterpret_cast<const Quad *>(in + off[1]);
    Quad x[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t q = lane + i * kWave;
      if (q < n_quads) x[i] = src[q];
    }
    if (addend != nullptr) {
      const Quad *add = reinterpret_cast<const Quad *>(addend + off[5]);
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        const uint32_t q = lane + i * kWave;
        if (q < n_quads) {
          const Quad y = add[q];
#pragma unroll
          for (int k = 0; k < 4; ++k) x[i].v[k] = x[i].v[k] + y.v[k];
        }
      }
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t q = lane + i * kWave;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (q >= n_quads) x[i].v[k] = 0.0f;
        s += x[i].v[k];
      }
    }
    s = WaveReduce(s, SumOp{});
    if (stale_scratch) s += scratch[off[4]];
    const float mean = s / n;
    float v = 0.0f;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t q = lane + i * kWave;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        x[i].v[k] = q < n_quads ? x[i].v[k] - mean : 0.0f;
        v += x[i].v[k] * x[i].v[k];
      }
    }
    v = WaveReduce(v, SumOp{});
    const float inv = 1.0f / sqrtf(v / n + eps);
    Quad *dst = reinterpret_cast<Quad *>(out + off[0]);
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t q = lane + i * kWave;
      if (q < n_quads) {
        const Quad g = gq[q], b = bq[q];
        Quad r;
#pragma unroll
        for (int k = 0; k < 4; ++k) r.v[k] = (x[i].v[k] * inv) * g.v[k] + b.v[k];
        StoreMaybeStreaming(dst + q, r, a.streaming != 0);
      }
    }
  }
}

// Any length / any axis stride: lanes of a block stride the row three times.
__global__ __launch_bounds__(kBlock) void LayerNormRowLoop(RowArgs<6> a, float *__restrict__ out,
                                                           const float *__restrict__ in,
                                                           const float *__restrict__ scale,
                                                           const float *__restrict__ bias,
                                                           const float *__restrict__ scratch, float eps,
                                                           int stale_scratch, const float *__restrict__ addend) {
  __shared__ float smem[kBlock / kWave];
  int32_t off[6];
  RowOffsets<6>(a.outer, blockIdx.x, off);
  const float *src = in + off[1];
  const int32_t si = a.axis_stride[1], so = a.axis_stride[0], sg = a.axis_stride[2], sb = a.axis_stride[3];
  const int32_t sy = a.axis_stride[5];
  auto at = [&](uint32_t j) {
    const int32_t jj = static_cast<int32_t>(j);
    return addend != nullptr ? src[jj * si] + addend[off[5] + jj * sy] : src[jj * si];
  };
  const float n = static_cast<float>(a.len);
  float s = 0.0f;
  for (uint32_t j = threadIdx.x; j < a.len; j += kBlock) s += at(j);
  s = BlockReduce<kBlock / kWave>(s, SumOp{}, smem);
  if (stale_scratch) s += scratch[off[4]];
  const float mean = s / n;
  float v = 0.0f;
  for (uint32_t j = threadIdx.x; j < a.len; j += kBlock) {
    const float d = at(j) - mean;
    v += d * d;
  }
  v = BlockReduce<kBlock / kWave>(v, SumOp{}, smem);
  const float inv = 1.0f / sqrtf(v / n + eps);
  float *dst = out + off[0];
  const float *g = scale + off[2];
  const float *b = bias + off[3];
  for (uint32_t j = threadIdx.x; j < a.len; j += kBlock) {
    const int32_t jj = static_cast<int32_t>(j);
    dst[jj * so] = ((at(j) - mean) * inv) * g[jj * sg] + b[jj * sb];
  }
}

// One lane per row (strided axis, many rows).
__global__ __launch_bounds__(kBlock) void LayerNormColumn(RowArgs<6> a, float *__restrict__ out,
                                                          const float *__restrict__ in,
                                                          const float *__restrict__ scale,
                                                          const float *__restrict__ bias,
                                                          const float *__restrict__ scratch, float eps,
                                                          int stale_scratch, const float *__restrict__ addend) {
  const uint32_t row = blockIdx.x * kBlock + threadIdx.x;
  if (row >= a.n_rows) return;
  int32_t off[6];
  RowOffsets<6>(a.outer, row, off);
  const float *src = in + off[1];
  const int32_t si = a.axis_stride[1], so = a.axis_stride[0], sg = a.axis_stride[2], sb = a.axis_stride[3];
  const int32_t sy = a.axis_stride[5];
  auto at = [&](uint32_t j) {
    const int32_t jj = static_cast<int32_t>(j);
    return addend != nullptr ? src[jj * si] + addend[off[5] + jj * sy] : src[jj * si];
  };
  const float n = static_cast<float>(a.len);
  float s = stale_scratch ? scratch[off[4]] : 0.0f;
  for (uint32_t j = 0; j < a.len; ++j) s += at(j);
  const float mean = s / n;
  float v = 0.0f;
  for (uint32_t j = 0; j < a.len; ++j) {
    const float d = at(j) - mean;
    v += d * d;
  }
  const float inv = 1.0f / sqrtf(v / n + eps);
  float *dst = out + off[0];
  const float *g = scale + off[2];
  const float *b = bias + off[3];
  for (uint32_t j = 0; j < a.len; ++j) {
    const int32_t jj = static_cast<int32_t>(j);
    dst[jj * so] = ((at(j) - mean) * inv) * g[jj * sg] + b[jj * sb];
  }
}

// ---- ReduceMean ---------------------------------------------------------------

struct ReduceArgs {
  NestArgs<2> outer;   // kept dims: operand 0 = output, 1 = input
  NestArgs<1> inner;   // reduced dims of the input
  uint32_t n_out;
  uint32_t n_red;
  float divisor;
};

__device__ __forceinline__ int32_t InnerOffset(const NestArgs<1> &a, uint32_t idx) {
  int32_t off[1] = {0};
  a.AddOffsets(idx, off);
  return off[0];
}

// One wave per output element.
__global__ __launch_bounds__(kBlock) void ReduceMeanWave(ReduceArgs a, float *__restrict__ out,
                                                         const float *__restrict__ in) {
  const uint32_t lane = threadIdx.x % kWave;
  const uint32_t o = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (o >= a.n_out) return;
  int32_t off[2];
  RowOffsets<2>(a.outer, o, off);
  const float *src = in + off[1];
  float s = 0.0f;
  for (uint32_t j = lane; j < a.n_red; j += kWave) s += src[InnerOffset(a.inner, j)];
  s = WaveReduce(s, SumOp{});
  if (lane == 0) out[off[0]] = s / a.divisor;
}

// The reduced dims are one unit-stride run: WAVES waves per output element (1, or the 4 of a workgroup when
// there are few outputs with long runs), 128-bit loads where the run starts on a 16-byte boundary, four
// independent partial sums per lane.
template <int WAVES>
__global__ __launch_bounds__(kBlock) void ReduceMeanRun(ReduceArgs a, float *__restrict__ out,
                                                        const float *__restrict__ in) {
  __shared__ float part[kBlock / kWave];
  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const uint32_t o = WAVES == 1 ? blockIdx.x * (kBlock / kWave) + wave : blockIdx.x;
  const bool active = o < a.n_out;
  int32_t off[2] = {0, 0};
  if (active) RowOffsets<2>(a.outer, o, off);
  const float *src = in + off[1];
  const uint32_t t = WAVES == 1 ? lane : threadIdx.x, nt = WAVES * kWave;
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  if (active) {
    uint32_t head = static_cast<uint32_t>((16 - (reinterpret_cast<uintptr_t>(src) & 15)) & 15) / 4;  // elements up to the boundary
    if (head > a.n_red) head = a.n_red;
    if (t < head) s0 += src[t];
    const uint32_t n4 = (a.n_red - head) / 4;
    const float *body = src + head;
    uint32_t j = t;
    // (eight loads in flight per lane while the run is long enough, then four, then one)
    for (; j + 7 * nt < n4; j += 8 * nt) {
      float4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const float4 *>(body + 4 * (j + u * nt));
      s0 += (v[0].x + v[0].y) + (v[0].z + v[0].w);
      s1 += (v[1].x + v[1].y) + (v[1].z + v[1].w);
      s2 += (v[2].x + v[2].y) + (v[2].z + v[2].w);
      s3 += (v[3].x + v[3].y) + (v[3].z + v[3].w);
      s0 += (v[4].x + v[4].y) + (v[4].z + v[4].w);
      s1 += (v[5].x + v[5].y) + (v[5].z + v[5].w);
      s2 += (v[6].x + v[6].y) + (v[6].z + v[6].w);
      s3 += (v[7].x + v[7].y) + (v[7].z + v[7].w);
    }
    for (; j + 3 * nt < n4; j += 4 * nt) {
      const float4 v0 = *reinterpret_cast<const float4 *>(body + 4 * j);
      const float4 v1 = *reinterpret_cast<const float4 *>(body + 4 * (j + nt));
      const float4 v2 = *reinterpret_cast<const float4 *>(body + 4 * (j + 2 * nt));
      const float4 v3 = *reinterpret_cast<const float4 *>(body + 4 * (j + 3 * nt));
      s0 += (v0.x + v0.y) + (v0.z + v0.w);
      s1 += (v1.x + v1.y) + (v1.z + v1.w);
      s2 += (v2.x + v2.y) + (v2.z + v2.w);
      s3 += (v3.x + v3.y) + (v3.z + v3.w);
    }
    for (; j < n4; j += nt) {
      const float4 v = *reinterpret_cast<const float4 *>(body + 4 * j);
      s0 += (v.x + v.y) + (v.z + v.w);
    }
    const uint32_t tail = head + 4 * n4;
    if (tail + t < a.n_red) s1 += src[tail + t];
  }
  float s = WaveReduce((s0 + s1) + (s2 + s3), SumOp{});
  if constexpr (WAVES == 1) {
    if (active && lane == 0) out[off[0]] = s / a.divisor;
  } else {
    if (lane == 0) part[wave] = s;
    __syncthreads();
    if (threadIdx.x == 0 && active) out[off[0]] = (((part[0] + part[1]) + part[2]) + part[3]) / a.divisor;
  }
}

// One lane per output element.
__global__ __launch_bounds__(kBlock) void ReduceMeanThread(ReduceArgs a, float *__restrict__ out,
                                                           const float *__restrict__ in) {
  const uint32_t o = blockIdx.x * kBlock + threadIdx.x;
  if (o >= a.n_out) return;
  int32_t off[2];
  RowOffsets<2>(a.outer, o, off);
  const float *src = in + off[1];
  float s = 0.0f;
  for (uint32_t j = 0; j < a.n_red; ++j) s += src[InnerOffset(a.inner, j)];
  out[off[0]] = s / a.divisor;
}

}  // namespace
}  // namespace fl

using namespace fl;

namespace fl {
namespace {

// ---- softmax over a short vector, then a matrix-vector product with it ------------------------------------------
// out[b, m] = sum_k a[b, m, k] * softmax_k(v[b, :])  (the per-position kernel of a span-based dynamic
// convolution: a handful of taps, softmaxed, applied to a window of values).  One lane per (b, m); the K <= 16
// logits of batch b are read by every lane of that batch (served by the cache) and normalised in registers.
constexpr int kMatVecMaxK = 16;

struct SoftmaxMatVecArgs {
  uint32_t n_items, rows;  // B * M, M
  FastDiv div_rows;
  int32_t k;
  int32_t a_b, a_m, a_k, v_b, v_k, out_b, out_m;  // element strides
  // the output's batch dim in two parts: batch b lies at (b / inner) * out_outer + (b % inner) * out_b
  FastDiv div_inner;
  int32_t out_outer;
};

__global__ __launch_bounds__(kBlock) void SoftmaxMatVecKernel(SoftmaxMatVecArgs p, float *__restrict__ out,
                                                              const float *__restrict__ a, const float *__restrict__ v) {
  const uint32_t item = blockIdx.x * kBlock + threadIdx.x;
  if (item >= p.n_items) return;
  uint32_t b, m;
  p.div_rows.DivMod(item, b, m);
  const float *logits = v + static_cast<int64_t>(b) * p.v_b;
  const float *row = a + static_cast<int64_t>(b) * p.a_b + static_cast<int64_t>(m) * p.a_m;
  float x[kMatVecMaxK], w[kMatVecMaxK];
  float top = -__FLT_MAX__;
#pragma unroll
  for (int t = 0; t < kMatVecMaxK; ++t) {
    x[t] = t < p.k ? logits[t * p.v_k] : -__FLT_MAX__;
    w[t] = t < p.k ? row[t * p.a_k] : 0.0f;
    top = fmaxf(top, x[t]);
  }
  float sum = 0.0f;
#pragma unroll
  for (int t = 0; t < kMatVecMaxK; ++t) {
    x[t] = t < p.k ? expf(x[t] - top) : 0.0f;
    sum += x[t];
  }
  float acc = 0.0f;
#pragma unroll
  for (int t = 0; t < kMatVecMaxK; ++t) acc += w[t] * (x[t] / sum);
  uint32_t b_outer, b_inner;
  p.div_inner.DivMod(b, b_outer, b_inner);
  out[static_cast<int64_t>(b_outer) * p.out_outer + static_cast<int64_t>(b_inner) * p.out_b + static_cast<int64_t>(m) * p.out_m] = acc;
}

}  // namespace
}  // namespace fl

extern "C" {

static int SoftmaxImpl(const fl_tensor *in, const fl_tensor *mask, float div, const fl_tensor *out, int64_t axis,
                       void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (in->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  if (!SameShape(in, out)) return FL_ERR_SHAPE;
  if (axis < 0 || axis >= in->rank) return FL_ERR_ATTR;  // reference normalises before the kernel
  int64_t strides[3][kMaxRank];
  for (int i = 0; i < in->rank; ++i) {
    strides[0][i] = out->strides[i];
    strides[1][i] = in->strides[i];
    strides[2][i] = 0;
  }
  SoftmaxPre pre{nullptr, 1.0f};
  if (mask != nullptr) {
    FL_CHECK(CheckView(mask));
    if (mask->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    FL_CHECK(BroadcastStrides(mask, in->rank, in->shape, strides[2]));
    pre.mask = static_cast<const float *>(mask->base);
    pre.div = div;
  }
  RowArgs<3> a = MakeRowArgs<3>(in->rank, in->shape, static_cast<int>(axis), strides);
  float *o = static_cast<float *>(out->base);
  const float *x = static_cast<const float *>(in->base);
  hipStream_t s = AsStream(stream);
  const bool row_contig = (a.axis_stride[0] == 1 && a.axis_stride[1] == 1) || a.len == 1;
  const bool many_rows = static_cast<int64_t>(a.n_rows) * a.len >= kManyRowsElements && a.len % 4 == 0 && a.len >= 32 &&
                         a.len <= 1024 && RowsVectorisable(out->base, in->rank, in->shape, static_cast<int>(axis), strides[0]) &&
                         RowsVectorisable(in->base, in->rank, in->shape, static_cast<int>(axis), strides[1]);
  if (many_rows) {
    auto blocks = [&](uint32_t lanes) { return dim3((a.n_rows + kBlock / lanes - 1) / (kBlock / lanes)); };
    if (a.len <= 64) {
      FL_LAUNCH((SoftmaxRowVec<8, 2>), blocks(8), dim3(kBlock), 0, s, a, o, x, pre);
    } else if (a.len <= 128) {
      FL_LAUNCH((SoftmaxRowVec<16, 2>), blocks(16), dim3(kBlock), 0, s, a, o, x, pre);
    } else if (a.len <= 256) {
      FL_LAUNCH((SoftmaxRowVec<16, 4>), blocks(16), dim3(kBlock), 0, s, a, o, x, pre);
    } else if (a.len <= 512) {
      FL_LAUNCH((SoftmaxRowVec<32, 4>), blocks(32), dim3(kBlock), 0, s, a, o, x, pre);
    } else {
      FL_LAUNCH((SoftmaxRowVec<64, 4>), blocks(64), dim3(kBlock), 0, s, a, o, x, pre);
    }
  } else if (row_contig && a.len > 16) {
    const uint32_t wave_blocks = (a.n_rows + kBlock / kWave - 1) / (kBlock / kWave);
    if (a.len <= 64) {
      FL_LAUNCH(SoftmaxRowWave<1>, dim3(wave_blocks), dim3(kBlock), 0, s, a, o, x, pre);
    } else if (a.len <= 128) {
      FL_LAUNCH(SoftmaxRowWave<2>, dim3(wave_blocks), dim3(kBlock), 0, s, a, o, x, pre);
    } else if (a.len <= 256) {
      FL_LAUNCH(SoftmaxRowWave<4>, dim3(wave_blocks), dim3(kBlock), 0, s, a, o, x, pre);
    } else if (a.len <= 512) {
      FL_LAUNCH(SoftmaxRowWave<8>, dim3(wave_blocks), dim3(kBlock), 0, s, a, o, x, pre);
    } else if (a.len <= 1024) {
      FL_LAUNCH(SoftmaxRowWave<16>, dim3(wave_blocks), dim3(kBlock), 0, s, a, o, x, pre);
    } else if (a.len <= 8 * kBlock) {
      FL_LAUNCH(SoftmaxRowBlockCached<8>, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, pre);
    } else if (a.len <= 16 * kBlock) {
      FL_LAUNCH(SoftmaxRowBlockCached<16>, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, pre);
    } else if (a.len <= 32 * kBlock) {
      FL_LAUNCH(SoftmaxRowBlockCached<32>, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, pre);
    } else {
      FL_LAUNCH(SoftmaxRowBlock, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, pre);
    }
  } else {
    FL_LAUNCH(SoftmaxColumn, dim3((a.n_rows + kBlock - 1) / kBlock), dim3(kBlock), 0, s, a, o, x, pre);
  }
  return LaunchStatus();
}

int fluidml_hip_softmax(const fl_tensor *in, const fl_tensor *out, void *scratch, size_t scratch_bytes, int64_t axis,
                        void *stream) {
  (void)scratch;
  (void)scratch_bytes;
  return SoftmaxImpl(in, nullptr, 1.0f, out, axis, stream);
}

int fluidml_hip_div_add_softmax(const fl_tensor *in, double div, const fl_tensor *mask, const fl_tensor *out,
                                int64_t axis, void *stream) {
  if (mask == nullptr) return FL_ERR_NULL;
  return SoftmaxImpl(in, mask, static_cast<float>(div), out, axis, stream);
}

static int LayerNormImpl(const fl_tensor *in, const fl_tensor *addend, const fl_tensor *scale, const fl_tensor *bias,
                         const fl_tensor *out, void *scratch, size_t scratch_bytes, int64_t axis, double epsilon,
                         uint32_t flags, void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(scale));
  FL_CHECK(CheckView(bias));
  FL_CHECK(CheckView(out));
  if (in->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32 || scale->dtype != FL_FLOAT32 || bias->dtype != FL_FLOAT32)
    return FL_ERR_DTYPE;
  if (!SameShape(in, out)) return FL_ERR_SHAPE;
  if (axis < 0) axis += in->rank;  // reference flow/node.cpp:931-933
  if (axis < 0 || axis >= in->rank) return FL_ERR_ATTR;
  const int stale = (flags & FL_REF_LN_STALE_SCRATCH) ? 1 : 0;
  int64_t strides[6][kMaxRank];
  FL_CHECK(BroadcastStrides(scale, in->rank, in->shape, strides[2]));
  FL_CHECK(BroadcastStrides(bias, in->rank, in->shape, strides[3]));
  const float *y = nullptr;
  if (addend != nullptr) {
    FL_CHECK(CheckView(addend));
    if (addend->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    FL_CHECK(BroadcastStrides(addend, in->rank, in->shape, strides[5]));
    y = static_cast<const float *>(addend->base);
  } else {
    for (int i = 0; i < in->rank; ++i) strides[5][i] = 0;
  }
  // scratch: dense row-major tensor of the input shape with axis -> 1
  int64_t acc = 1, rows = 1;
  for (int i = in->rank - 1; i >= 0; --i) {
    strides[0][i] = out->strides[i];
    strides[1][i] = in->strides[i];
    if (i == axis) {
      strides[4][i] = 0;
    } else {
      strides[4][i] = acc;
      acc *= in->shape[i];
      rows *= in->shape[i];
    }
  }
  if (stale) {
    if (scratch == nullptr) return FL_ERR_NULL;
    if (scratch_bytes < static_cast<size_t>(rows) * sizeof(float)) return FL_ERR_SCRATCH;
  }
  RowArgs<6> a = MakeRowArgs<6>(in->rank, in->shape, static_cast<int>(axis), strides);
  float *o = static_cast<float *>(out->base);
  const float *x = static_cast<const float *>(in->base);
  const float *g = static_cast<const float *>(scale->base);
  const float *b = static_cast<const float *>(bias->base);
  const float *sc = static_cast<const float *>(scratch);
  const float eps = static_cast<float>(epsilon);
  hipStream_t s = AsStream(stream);
  const bool row_contig = a.axis_stride[0] == 1 && a.axis_stride[1] == 1;
  const int ax = static_cast<int>(axis);
  const bool many_rows = static_cast<int64_t>(a.n_rows) * a.len >= kManyRowsElements && a.len % 4 == 0 && a.len >= 256 &&
                         a.len <= 16 * 256 && RowsVectorisable(out->base, in->rank, in->shape, ax, strides[0]) &&
                         RowsVectorisable(in->base, in->rank, in->shape, ax, strides[1]) &&
                         (y == nullptr || RowsVectorisable(y, in->rank, in->shape, ax, strides[5])) &&
                         RowInvariant(in->rank, in->shape, ax, strides[2]) && RowInvariant(in->rank, in->shape, ax, strides[3]);
  if (many_rows) {
    // eight workgroups per compute unit at most: each keeps its copy of scale and bias for many rows
    const dim3 wave_grid(std::min<uint32_t>((a.n_rows + kBlock / kWave - 1) / (kBlock / kWave), 256 * 8));
    const size_t lds_bytes = 2 * static_cast<size_t>(a.len) * sizeof(float);
    const uint32_t items = (a.len + 255) / 256;
#define FL_LN_VEC(ITEMS) \
  FL_LAUNCH(LayerNormRowVec<ITEMS>, wave_grid, dim3(kBlock), lds_bytes, s, a, o, x, g, b, sc, eps, stale, y)
    if (items <= 1) {
      FL_LN_VEC(1);
    } else if (items <= 2) {
      FL_LN_VEC(2);
    } else if (items <= 3) {
      FL_LN_VEC(3);
    } else if (items <= 4) {
      FL_LN_VEC(4);
    } else if (items <= 6) {
      FL_LN_VEC(6);
    } else if (items <= 8) {
      FL_LN_VEC(8);
    } else if (items <= 12) {
      FL_LN_VEC(12);
    } else {
      FL_LN_VEC(16);
    }
#undef FL_LN_VEC
  } else if (row_contig && a.len > 64) {
    const dim3 wave_grid((a.n_rows + kBlock / kWave - 1) / (kBlock / kWave));
    if (a.len <= 4 * kWave) {
      FL_LAUNCH(LayerNormRowWave<4>, wave_grid, dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    } else if (a.len <= 8 * kWave && a.n_rows >= 1024) {
      FL_LAUNCH(LayerNormRowWave<8>, wave_grid, dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    } else if (a.len <= 12 * kWave && a.n_rows >= 1024) {
      FL_LAUNCH(LayerNormRowWave<12>, wave_grid, dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    } else if (a.len <= 16 * kWave && a.n_rows >= 1024) {
      FL_LAUNCH(LayerNormRowWave<16>, wave_grid, dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    } else if (a.len <= kBlock) {
      FL_LAUNCH(LayerNormRowBlock<1>, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    } else if (a.len <= 2 * kBlock) {
      FL_LAUNCH(LayerNormRowBlock<2>, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    } else if (a.len <= 4 * kBlock) {
      FL_LAUNCH(LayerNormRowBlock<4>, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    } else if (a.len <= 8 * kBlock) {
      FL_LAUNCH(LayerNormRowBlock<8>, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    } else if (a.len <= 16 * kBlock) {
      FL_LAUNCH(LayerNormRowBlock<16>, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    } else if (a.len <= 32 * kBlock) {
      FL_LAUNCH(LayerNormRowBlock<32>, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    } else {
      FL_LAUNCH(LayerNormRowLoop, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
    }
  } else if (a.n_rows >= 4096 || a.len <= 64) {
    FL_LAUNCH(LayerNormColumn, dim3((a.n_rows + kBlock - 1) / kBlock), dim3(kBlock), 0, s, a, o, x, g, b, sc,
                       eps, stale, y);
  } else {
    FL_LAUNCH(LayerNormRowLoop, dim3(a.n_rows), dim3(kBlock), 0, s, a, o, x, g, b, sc, eps, stale, y);
  }
  return LaunchStatus();
}

int fluidml_hip_layer_normalization_constant_scale_bias(const fl_tensor *in, const fl_tensor *scale,
                                                        const fl_tensor *bias, const fl_tensor *out, void *scratch,
                                                        size_t scratch_bytes, int64_t axis, double epsilon,
                                                        uint32_t flags, void *stream) {
  return LayerNormImpl(in, nullptr, scale, bias, out, scratch, scratch_bytes, axis, epsilon, flags, stream);
}

int fluidml_hip_add_layer_normalization(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *scale,
                                        const fl_tensor *bias, const fl_tensor *out, int64_t axis, double epsilon,
                                        void *stream) {
  if (rhs == nullptr) return FL_ERR_NULL;
  return LayerNormImpl(lhs, rhs, scale, bias, out, nullptr, 0, axis, epsilon, 0, stream);
}

namespace {
bool DenseRowMajor(const fl_tensor *t) {
  int64_t want = 1;
  for (int i = t->rank - 1; i >= 0; --i) {
    if (t->shape[i] != 1 && t->strides[i] != want) return false;
    want *= t->shape[i];
  }
  return true;
}
int64_t Elements(const fl_tensor *t) {
  int64_t n = 1;
  for (int i = 0; i < t->rank; ++i) n *= t->shape[i];
  return n;
}
// `t` as an addend of `out` [rows..., len]: its dims, aligned at the right, equal out's, with nothing but ones in
// front; *rows = how many rows it holds (it repeats after them)
int AddendRows(const fl_tensor *t, const fl_tensor *out, uint32_t *rows) {
  FL_CHECK(CheckView(t));
  if (t->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  if (t->rank > out->rank || t->rank < 1 || !DenseRowMajor(t)) return FL_ERR_UNSUPPORTED;
  bool ones = false;
  for (int i = 1; i <= out->rank; ++i) {
    const int64_t have = i <= t->rank ? t->shape[t->rank - i] : 1;
    const int64_t want = out->shape[out->rank - i];
    if (!ones && have == want) continue;
    if (have != 1 || i == 1) return FL_ERR_UNSUPPORTED;  // broadcast along the row or between kept dims
    ones = true;
  }
  *rows = static_cast<uint32_t>(Elements(t) / out->shape[out->rank - 1]);
  return FL_OK;
}
}  // namespace

int fluidml_hip_gather_add_layer_normalization(const fl_tensor *indices0, const fl_tensor *data0,
                                               const fl_tensor *indices1, const fl_tensor *second,
                                               const fl_tensor *third, const fl_tensor *scale, const fl_tensor *bias,
                                               const fl_tensor *out, double epsilon, void *stream) {
  if (!indices0 || !data0 || !second || !scale || !bias || !out) return FL_ERR_NULL;
  for (const fl_tensor *t : {indices0, data0, second, scale, bias, out}) FL_CHECK(CheckView(t));
  if (indices1 != nullptr) FL_CHECK(CheckView(indices1));
  if (indices0->dtype != FL_INT64 || (indices1 != nullptr && indices1->dtype != FL_INT64)) return FL_ERR_DTYPE;
  if (data0->dtype != FL_FLOAT32 || second->dtype != FL_FLOAT32 || scale->dtype != FL_FLOAT32 ||
      bias->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32)
    return FL_ERR_DTYPE;
  if (data0->rank != 2 || out->rank != indices0->rank + 1 || out->rank < 1) return FL_ERR_RANK;
  const int64_t len = data0->shape[1];
  for (int i = 0; i < indices0->rank; ++i) {
    if (out->shape[i] != indices0->shape[i]) return FL_ERR_SHAPE;
  }
  if (out->shape[out->rank - 1] != len || Elements(scale) != len || Elements(bias) != len) return FL_ERR_SHAPE;
  if (!DenseRowMajor(indices0) || !DenseRowMajor(data0) || !DenseRowMajor(out) || !DenseRowMajor(scale) ||
      !DenseRowMajor(bias))
    return FL_ERR_UNSUPPORTED;
  if (len < 1 || len > FL_GATHER_LAYER_NORM_MAX_LEN) return FL_ERR_UNSUPPORTED;
  const int64_t rows = Elements(indices0);
  if (rows > INT32_MAX) return FL_ERR_TOO_LARGE;
  EmbedArgs a{};
  a.len = static_cast<uint32_t>(len);
  a.rows0 = data0->shape[0];
  a.second_rows = a.third_rows = 1;
  if (indices1 != nullptr) {
    if (second->rank != 2 || second->shape[1] != len || !DenseRowMajor(second) || !DenseRowMajor(indices1))
      return FL_ERR_UNSUPPORTED;
    if (indices1->rank != indices0->rank) return FL_ERR_RANK;
    for (int i = 0; i < indices0->rank; ++i) {
      if (indices1->shape[i] != indices0->shape[i]) return FL_ERR_SHAPE;
    }
    a.rows1 = second->shape[0];
  } else {
    FL_CHECK(AddendRows(second, out, &a.second_rows));
  }
  if (third != nullptr) FL_CHECK(AddendRows(third, out, &a.third_rows));
  if (rows == 0) return FL_OK;
  hipStream_t s = AsStream(stream);
  float *o = static_cast<float *>(out->base);
  const int64_t *i0 = static_cast<const int64_t *>(indices0->base);
  const int64_t *i1 = indices1 != nullptr ? static_cast<const int64_t *>(indices1->base) : nullptr;
  const float *d0 = static_cast<const float *>(data0->base), *d1 = static_cast<const float *>(second->base);
  const float *d2 = third != nullptr ? static_cast<const float *>(third->base) : nullptr;
  const float *g = static_cast<const float *>(scale->base), *b = static_cast<const float *>(bias->base);
  const float eps = static_cast<float>(epsilon);
  const dim3 grid(static_cast<uint32_t>(rows));
#define FL_EMBED(ITEMS) \
  FL_LAUNCH(EmbeddingLayerNormKernel<ITEMS>, grid, dim3(kBlock), 0, s, a, o, i0, d0, i1, d1, d2, g, b, eps)
  if (len <= kBlock) {
    FL_EMBED(1);
  } else if (len <= 2 * kBlock) {
    FL_EMBED(2);
  } else if (len <= 4 * kBlock) {
    FL_EMBED(4);
  } else {
    FL_EMBED(8);
  }
#undef FL_EMBED
  return LaunchStatus();
}

int fluidml_hip_gather_constant_data_tensor_stats(const fl_tensor *indices, const fl_tensor *data, const fl_tensor *out,
                                                  float *stats_out, void *stream) {
  if (!indices || !data || !out || !stats_out) return FL_ERR_NULL;
  for (const fl_tensor *t : {indices, data, out}) FL_CHECK(CheckView(t));
  if (indices->dtype != FL_INT64 || data->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  if (data->rank != 2 || out->rank != indices->rank + 1) return FL_ERR_RANK;
  for (int i = 0; i < indices->rank; ++i) {
    if (out->shape[i] != indices->shape[i]) return FL_ERR_SHAPE;
  }
  if (out->shape[out->rank - 1] != data->shape[1]) return FL_ERR_SHAPE;
  if (!DenseRowMajor(indices) || !DenseRowMajor(data) || !DenseRowMajor(out)) return FL_ERR_UNSUPPORTED;
  const int64_t rows = Elements(indices);
  if (rows > INT32_MAX || data->shape[1] > INT32_MAX) return FL_ERR_TOO_LARGE;
  if (rows == 0 || data->shape[1] == 0) return FL_OK;
  FL_LAUNCH(GatherStatsKernel, dim3(static_cast<uint32_t>(rows)), dim3(kBlock), 0, AsStream(stream),
            static_cast<uint32_t>(data->shape[1]), data->shape[0], static_cast<float *>(out->base),
            static_cast<const int64_t *>(indices->base), static_cast<const float *>(data->base), stats_out);
  return LaunchStatus();
}

int fluidml_hip_reduce_mean(const fl_tensor *in, const fl_tensor *out, const int64_t *axes, int32_t n_axes,
                            void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (in->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  if (in->rank != out->rank) return FL_ERR_UNSUPPORTED;  // keepdims=0: unreachable in reference reduce_mean.cpp:56-62
  if (n_axes < 0 || (n_axes > 0 && axes == nullptr)) return FL_ERR_ATTR;
  bool reduced[kMaxRank] = {};
  for (int k = 0; k < n_axes; ++k) {
    if (axes[k] < 0 || axes[k] >= in->rank) return FL_ERR_ATTR;
    reduced[axes[k]] = true;
  }
  LoopNest outer, inner;
  outer.n_operands = 2;
  inner.n_operands = 1;
  int64_t divisor = 1;
  for (int i = 0; i < in->rank; ++i) {
    if (reduced[i]) {
      if (out->shape[i] != 1) return FL_ERR_SHAPE;
      divisor *= in->shape[i];
      inner.shape[inner.rank] = in->shape[i];
      inner.strides[0][inner.rank] = in->strides[i];
      ++inner.rank;
    } else {
      if (out->shape[i] != in->shape[i]) return FL_ERR_SHAPE;
      outer.shape[outer.rank] = in->shape[i];
      outer.strides[0][outer.rank] = out->strides[i];
      outer.strides[1][outer.rank] = in->strides[i];
      ++outer.rank;
    }
  }
  outer.Canonicalise();
  inner.Canonicalise();
  ReduceArgs a;
  a.outer = MakeNestArgs<2>(outer);
  a.inner = MakeNestArgs<1>(inner);
  int64_t n_out = 1, n_red = 1;
  for (int i = 0; i < outer.rank; ++i) n_out *= outer.shape[i];
  for (int i = 0; i < inner.rank; ++i) n_red *= inner.shape[i];
  a.n_out = static_cast<uint32_t>(n_out);
  a.n_red = static_cast<uint32_t>(n_red);
  a.divisor = static_cast<float>(divisor);
  float *o = static_cast<float *>(out->base);
  const float *x = static_cast<const float *>(in->base);
  hipStream_t s = AsStream(stream);
  const bool inner_contig = inner.strides[0][inner.rank - 1] == 1;
  if (inner.rank == 1 && inner_contig && n_red >= 64) {
    if (n_out <= 512 && n_red >= 1024) {
      FL_LAUNCH(ReduceMeanRun<kBlock / kWave>, dim3(a.n_out), dim3(kBlock), 0, s, a, o, x);
    } else {
      FL_LAUNCH(ReduceMeanRun<1>, dim3((a.n_out + kBlock / kWave - 1) / (kBlock / kWave)), dim3(kBlock), 0, s, a, o, x);
    }
  } else if ((inner_contig && n_red >= 32) || n_out < 1024) {
    FL_LAUNCH(ReduceMeanWave, dim3((a.n_out + kBlock / kWave - 1) / (kBlock / kWave)), dim3(kBlock), 0, s, a, o,
                       x);
  } else {
    FL_LAUNCH(ReduceMeanThread, dim3((a.n_out + kBlock - 1) / kBlock), dim3(kBlock), 0, s, a, o, x);
  }
  return LaunchStatus();
}

int fluidml_hip_softmax_matvec(const fl_tensor *a, const fl_tensor *logits, const fl_tensor *out, void *stream) {
  using namespace fl;
  FL_CHECK(CheckView(a));
  FL_CHECK(CheckView(logits));
  FL_CHECK(CheckView(out));
  if (a->dtype != FL_FLOAT32 || logits->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  if (a->rank != 3 || logits->rank != 3 || (out->rank != 3 && out->rank != 4)) return FL_ERR_RANK;
  const int64_t batch = a->shape[0], rows = a->shape[1], k = a->shape[2];
  const int split = out->rank - 3;  // 1: out is [outer, inner, rows, 1] with outer * inner batches
  const int64_t out_batch = split ? out->shape[0] * out->shape[1] : out->shape[0];
  if (logits->shape[0] != batch || logits->shape[1] != k || logits->shape[2] != 1 || out_batch != batch ||
      out->shape[split + 1] != rows || out->shape[split + 2] != 1 || (split && out->shape[1] < 1)) {
    return FL_ERR_SHAPE;
  }
  if (k > kMatVecMaxK) return FL_ERR_UNSUPPORTED;
  SoftmaxMatVecArgs p;
  p.n_items = static_cast<uint32_t>(batch * rows);
  p.rows = static_cast<uint32_t>(rows);
  p.div_rows = FastDiv(static_cast<uint32_t>(rows));
  p.k = static_cast<int32_t>(k);
  p.a_b = static_cast<int32_t>(a->strides[0]);
  p.a_m = static_cast<int32_t>(a->strides[1]);
  p.a_k = static_cast<int32_t>(a->strides[2]);
  p.v_b = static_cast<int32_t>(logits->strides[0]);
  p.v_k = static_cast<int32_t>(logits->strides[1]);
  p.out_b = static_cast<int32_t>(out->strides[split]);
  p.out_m = static_cast<int32_t>(out->strides[split + 1]);
  p.div_inner = FastDiv(static_cast<uint32_t>(split ? out->shape[1] : batch > 0 ? batch : 1));
  p.out_outer = split ? static_cast<int32_t>(out->strides[0]) : 0;
  FL_LAUNCH(SoftmaxMatVecKernel, dim3((p.n_items + kBlock - 1) / kBlock), dim3(kBlock), 0, AsStream(stream), p,
            static_cast<float *>(out->base), static_cast<const float *>(a->base), static_cast<const float *>(logits->base));
  return LaunchStatus();
}

}  // extern "C"
