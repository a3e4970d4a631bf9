// Elementwise and strided-copy kernels (HBM bound).
//
// One loop-nest engine serves every all-parallel linalg.generic of the
// reference (src/structure/kernel/kernel/{add,sub,mul,div,pow,erf,relu,clip,
// tanh,sqrt,neg,not,cast,equal,dropout,where,transpose,squeeze,unsqueeze,
// slice,concat,pad,add_div_erf_add_mul_mul,unsqueeze_sub_mul}.cpp): the host
// wrapper turns the kernel's affine maps into per-operand strides, the nest is
// canonicalised in the output's physical order, and the device walks it with
// 128-bit accesses when the innermost dimension is contiguous for every
// operand (or broadcast), falling back to scalar accesses otherwise.
#include "fl_common.h"

namespace fl {
namespace {

template <typename T, int N>
struct alignas(sizeof(T) * N) Vec {
  T v[N];
};

struct Empty {};

constexpr int kBlock = 256;
constexpr int kVec = 4;

// NIN inputs, operand 0 of the nest is the output.  `bcast` bit i set = input
// i is broadcast along the innermost dimension (scalar load, replicated); bit 31 set = the output is large
// enough to be written with non-temporal stores.
constexpr uint32_t kStreamingBit = 1u << 31;
template <int NIN, int VEC, typename TO, typename T0, typename T1, typename T2, typename Op>
__global__ __launch_bounds__(kBlock) void EwKernel(NestArgs<NIN + 1> a, uint32_t n_items, uint32_t bcast,
                                                   TO *__restrict__ out, const T0 *__restrict__ in0,
                                                   const T1 *__restrict__ in1, const T2 *__restrict__ in2, Op op) {
  const uint32_t stride = gridDim.x * kBlock;
  const bool streaming = (bcast & kStreamingBit) != 0;
  for (uint32_t item = blockIdx.x * kBlock + threadIdx.x; item < n_items; item += stride) {
    int32_t off[NIN + 1];
#pragma unroll
    for (int o = 0; o <= NIN; ++o) off[o] = 0;
    a.AddOffsets(item, off);

    if constexpr (VEC == 1) {
      T0 x0 = in0[off[1]];
      T1 x1{};
      T2 x2{};
      if constexpr (NIN >= 2) x1 = in1[off[2]];
      if constexpr (NIN >= 3) x2 = in2[off[3]];
      StoreMaybeStreaming(out + off[0], static_cast<TO>(op(x0, x1, x2)), streaming);
    } else {
      Vec<T0, VEC> v0;
      Vec<T1, VEC> v1;
      Vec<T2, VEC> v2;
      if (bcast & 1u) {
        const T0 s = in0[off[1]];
#pragma unroll
        for (int i = 0; i < VEC; ++i) v0.v[i] = s;
      } else {
        v0 = *reinterpret_cast<const Vec<T0, VEC> *>(in0 + off[1]);
      }
      if constexpr (NIN >= 2) {
        if (bcast & 2u) {
          const T1 s = in1[off[2]];
#pragma unroll
          for (int i = 0; i < VEC; ++i) v1.v[i] = s;
        } else {
          v1 = *reinterpret_cast<const Vec<T1, VEC> *>(in1 + off[2]);
        }
      }
      if constexpr (NIN >= 3) {
        if (bcast & 4u) {
          const T2 s = in2[off[3]];
#pragma unroll
          for (int i = 0; i < VEC; ++i) v2.v[i] = s;
        } else {
          v2 = *reinterpret_cast<const Vec<T2, VEC> *>(in2 + off[3]);
        }
      }
      Vec<TO, VEC> r;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        T1 x1{};
        T2 x2{};
        if constexpr (NIN >= 2) x1 = v1.v[i];
        if constexpr (NIN >= 3) x2 = v2.v[i];
        r.v[i] = op(v0.v[i], x1, x2);
      }
      StoreMaybeStreaming(reinterpret_cast<Vec<TO, VEC> *>(out + off[0]), r, streaming);
    }
  }
}

// Decide vector width, build device args, launch.
template <int NIN, typename TO, typename T0, typename T1, typename T2, typename Op>
int LaunchNest(LoopNest nest, void *out, const void *in0, const void *in1, const void *in2, Op op, hipStream_t stream) {
  nest.Canonicalise();
  int64_t total = 1;
  for (int i = 0; i < nest.rank; ++i) total *= nest.shape[i];
  if (total > INT32_MAX) return FL_ERR_TOO_LARGE;

  const void *ptrs[4] = {out, in0, in1, in2};
  const size_t sizes[4] = {sizeof(TO), sizeof(T0), sizeof(T1), sizeof(T2)};
  const int inner = nest.rank - 1;
  bool vec_ok = nest.shape[inner] % kVec == 0 && nest.strides[0][inner] == 1;
  uint32_t bcast = 0;
  for (int o = 0; o <= NIN && vec_ok; ++o) {
    const int64_t s = nest.strides[o][inner];
    if (s == 0 && o > 0) {
      bcast |= 1u << (o - 1);
    } else if (s != 1) {
      vec_ok = false;
      break;
    }
    if (!IsAligned(ptrs[o], sizes[o] * kVec) && s == 1) vec_ok = false;
    for (int d = 0; d < inner && vec_ok; ++d) {
      if (s == 1 && nest.strides[o][d] % kVec != 0) vec_ok = false;
    }
  }
  if (!vec_ok) bcast = 0;

  if (vec_ok) {
    nest.shape[inner] /= kVec;
    for (int o = 0; o <= NIN; ++o) nest.strides[o][inner] *= kVec;
  }
  const int64_t n_items = vec_ok ? total / kVec : total;
  NestArgs<NIN + 1> args = MakeNestArgs<NIN + 1>(nest);
  const int64_t blocks_needed = (n_items + kBlock - 1) / kBlock;
  // a large streaming launch is fastest with one item per lane (256 MiB copy: 8192 workgroups 5.5 TB/s,
  // 65536 workgroups 5.9 TB/s, with non-temporal stores 6.8 and 7.2 TB/s)
  const bool streaming = StreamingOutput(static_cast<size_t>(total) * sizeof(TO));
  const uint32_t grid = static_cast<uint32_t>(std::min<int64_t>(blocks_needed, streaming ? 256 * 256 : 256 * 32));
  if (streaming) bcast |= kStreamingBit;
  if (vec_ok) {
    FL_LAUNCH((EwKernel<NIN, kVec, TO, T0, T1, T2, Op>), dim3(grid), dim3(kBlock), 0, stream, args,
                       static_cast<uint32_t>(n_items), bcast, static_cast<TO *>(out), static_cast<const T0 *>(in0),
                       static_cast<const T1 *>(in1), static_cast<const T2 *>(in2), op);
  } else {
    FL_LAUNCH((EwKernel<NIN, 1, TO, T0, T1, T2, Op>), dim3(grid), dim3(kBlock), 0, stream, args,
                       static_cast<uint32_t>(n_items), bcast & kStreamingBit, static_cast<TO *>(out), static_cast<const T0 *>(in0),
                       static_cast<const T1 *>(in1), static_cast<const T2 *>(in2), op);
  }
  return LaunchStatus();
}

// ---- functors ---------------------------------------------------------------

template <typename T>
struct AddC {
  T c;
  __device__ T operator()(T x, Empty, Empty) const { return x + c; }
};
template <typename T>
struct RSubC {
  T c;
  __device__ T operator()(T x, Empty, Empty) const { return c - x; }
};
template <typename T>
struct MulC {
  T c;
  __device__ T operator()(T x, Empty, Empty) const { return x * c; }
};
struct DivC {
  float c;
  __device__ float operator()(float x, Empty, Empty) const { return x / c; }
};
struct PowC {
  float c;
  __device__ float operator()(float x, Empty, Empty) const { return powf(x, c); }
};
struct Erf {
  __device__ float operator()(float x, Empty, Empty) const { return erff(x); }
};
struct Relu {
  // arith.maximumf against 0 propagates NaN (reference relu.cpp:12-46)
  __device__ float operator()(float x, Empty, Empty) const { return x != x ? x : fmaxf(x, 0.0f); }
};
struct Clip {
  float lo, hi;
  __device__ float operator()(float x, Empty, Empty) const {
    return x != x ? x : fminf(fmaxf(x, lo), hi);
  }
};
struct Tanh {
  __device__ float operator()(float x, Empty, Empty) const { return tanhf(x); }
};
struct Sqrt {
  __device__ float operator()(float x, Empty, Empty) const { return sqrtf(x); }
};
struct Neg {
  __device__ float operator()(float x, Empty, Empty) const { return -x; }
};
struct Chain {
  fl_ew_program g;
  __device__ float operator()(float x, Empty, Empty) const { return RunChain(g, x); }
};
struct Not {
  __device__ uint8_t operator()(uint8_t x, Empty, Empty) const { return x ^ 1u; }
};
template <typename TO, typename TI>
struct Copy {
  __device__ TO operator()(TI x, Empty, Empty) const { return static_cast<TO>(x); }
};
struct EqC {
  int64_t c;
  __device__ uint8_t operator()(int64_t x, Empty, Empty) const { return x == c ? 1 : 0; }
};
template <typename T>
struct Add2 {
  __device__ T operator()(T a, T b, Empty) const { return a + b; }
};
template <typename T>
struct Sub2 {
  __device__ T operator()(T a, T b, Empty) const { return a - b; }
};
template <typename T>
struct Mul2 {
  __device__ T operator()(T a, T b, Empty) const { return a * b; }
};
struct Div2 {
  __device__ float operator()(float a, float b, Empty) const { return a / b; }
};
// a * b + c with the product rounded before the sum, as the two separate kernels round it
struct MulAdd3 {
  __device__ float operator()(float a, float b, float c) const {
#pragma clang fp contract(off)
    const float product = a * b;
    return product + c;
  }
};
// (a + b) + c, the two sums in the order of the two separate kernels
struct AddAdd3 {
  __device__ float operator()(float a, float b, float c) const { return (a + b) + c; }
};
struct WhereScalarY {
  float y;
  __device__ float operator()(uint8_t c, float x, Empty) const { return c ? x : y; }
};
struct WhereTensorY {
  __device__ float operator()(uint8_t c, float x, float y) const { return c ? x : y; }
};
struct Gelu {
  // t = x + b; t * (erf(t / c_div) + c_add) * c_mul, evaluated in the order of
  // reference add_div_erf_add_mul_mul.cpp:29-132: mul0 = t * (erf + c_add); out = mul0 * c_mul
  float c_div, c_add, c_mul;
  __device__ float operator()(float x, float b, Empty) const {
    const float t = x + b;
    return (t * (erff(t / c_div) + c_add)) * c_mul;
  }
};
struct SubMul {
  float c_sub, c_mul;
  __device__ float operator()(float x, Empty, Empty) const { return (c_sub - x) * c_mul; }
};

// ---- nest builders ----------------------------------------------------------

int IdentityNest(const fl_tensor *in, const fl_tensor *out, LoopNest *nest) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (!SameShape(in, out)) return FL_ERR_SHAPE;
  nest->rank = out->rank;
  nest->n_operands = 2;
  for (int i = 0; i < out->rank; ++i) {
    nest->shape[i] = out->shape[i];
    nest->strides[0][i] = out->strides[i];
    nest->strides[1][i] = in->strides[i];
  }
  return FL_OK;
}

int BroadcastNest(const fl_tensor *const *ins, int n_in, const fl_tensor *out, LoopNest *nest) {
  FL_CHECK(CheckView(out));
  nest->rank = out->rank;
  nest->n_operands = n_in + 1;
  for (int i = 0; i < out->rank; ++i) {
    nest->shape[i] = out->shape[i];
    nest->strides[0][i] = out->strides[i];
  }
  for (int k = 0; k < n_in; ++k) {
    FL_CHECK(CheckView(ins[k]));
    FL_CHECK(BroadcastStrides(ins[k], out->rank, out->shape, nest->strides[k + 1]));
  }
  return FL_OK;
}

template <typename TO, typename TI, typename Op>
int Unary(const LoopNest &nest, const fl_tensor *in, const fl_tensor *out, Op op, void *stream) {
  return LaunchNest<1, TO, TI, Empty, Empty>(nest, out->base, in->base, nullptr, nullptr, op, AsStream(stream));
}

template <typename Op>
int UnaryF32(const fl_tensor *in, const fl_tensor *out, Op op, void *stream) {
  LoopNest nest;
  FL_CHECK(IdentityNest(in, out, &nest));
  if (in->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  return Unary<float, float>(nest, in, out, op, stream);
}

template <typename T, typename Op>
int Binary(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, Op op, void *stream) {
  const fl_tensor *ins[2] = {lhs, rhs};
  LoopNest nest;
  FL_CHECK(BroadcastNest(ins, 2, out, &nest));
  return LaunchNest<2, T, T, T, Empty>(nest, out->base, lhs->base, rhs->base, nullptr, op, AsStream(stream));
}

// Copy whose fastest output dim is not the fastest input dim (a transposing layout change): 64x64 tiles go
// through LDS so that both the global reads (along the input's unit-stride dim) and the global writes (along
// the output's) are coalesced.  `outer` enumerates the remaining dims (operand 0 = out, 1 = in).
struct TiledCopyArgs {
  NestArgs<2> outer;
  uint32_t n_out_fast, n_in_fast;  // extents of the output-fast dim and of the input-fast dim
  int32_t in_stride_of_out_fast;   // input stride along the output-fast dim
  int32_t out_stride_of_in_fast;   // output stride along the input-fast dim
  uint32_t tiles_out_fast, tiles_in_fast;
  uint32_t streaming;  // 1 = non-temporal stores
};

__global__ __launch_bounds__(256) void TiledCopyKernel(TiledCopyArgs a, uint32_t *__restrict__ out,
                                                       const uint32_t *__restrict__ in) {
  __shared__ uint32_t tile[64][65];
  // Diagonal order: consecutive workgroups differ in BOTH tile coordinates.  Walking one coordinate alone makes
  // every resident workgroup read (or write) addresses that are equal modulo a row pitch, and a power-of-two
  // pitch then lands them all on the same few memory channels.
  const uint32_t t_of = blockIdx.x % a.tiles_out_fast;
  const uint32_t t_if = (blockIdx.x / a.tiles_out_fast + t_of) % a.tiles_in_fast;
  const bool streaming = a.streaming != 0;
  int32_t off2[2] = {0, 0};
  a.outer.AddOffsets(blockIdx.x / (a.tiles_out_fast * a.tiles_in_fast), off2);
  const int32_t off_out = off2[0], off_in = off2[1];
  const uint32_t of0 = t_of * 64, if0 = t_if * 64;
  const uint32_t lane = threadIdx.x % 64, row = threadIdx.x / 64;
  // read: lanes run along the input-fast dim
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const uint32_t jo = of0 + row + 4 * r, ji = if0 + lane;
    if (jo < a.n_out_fast && ji < a.n_in_fast) {
      tile[row + 4 * r][lane] = in[off_in + static_cast<int32_t>(jo) * a.in_stride_of_out_fast + static_cast<int32_t>(ji)];
    }
  }
  __syncthreads();
  // write: lanes run along the output-fast dim
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const uint32_t ji = if0 + row + 4 * r, jo = of0 + lane;
    if (jo < a.n_out_fast && ji < a.n_in_fast) {
      StoreMaybeStreaming(out + off_out + static_cast<int32_t>(ji) * a.out_stride_of_in_fast + static_cast<int32_t>(jo),
                          tile[lane][row + 4 * r], streaming);
    }
  }
}

// The same tile moved with 128-bit accesses on both sides (four values of a row per lane; LDS accesses stay
// 32-bit and conflict-free): both fast extents, the two cross strides and every outer stride are multiples of 4
// and both bases are 16-byte aligned.  [4096,16384] -> [16384,4096]: 3.6 TB/s with the kernel above, 4.3 TB/s
// with this one and 6.7 TB/s once its stores are non-temporal.
__global__ __launch_bounds__(256) void TiledCopyVecKernel(TiledCopyArgs a, uint32_t *__restrict__ out,
                                                          const uint32_t *__restrict__ in) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  __shared__ uint32_t tile[64][65];  // [input-fast][output-fast]
  const uint32_t t_of = blockIdx.x % a.tiles_out_fast, t_if = (blockIdx.x / a.tiles_out_fast) % a.tiles_in_fast;
  int32_t off2[2] = {0, 0};
  a.outer.AddOffsets(blockIdx.x / (a.tiles_out_fast * a.tiles_in_fast), off2);
  const int32_t off_out = off2[0], off_in = off2[1];
  const uint32_t of0 = t_of * 64, if0 = t_if * 64;
  const uint32_t quad = threadIdx.x % 16, row = threadIdx.x / 16;
  const bool streaming = a.streaming != 0;
  u32x4 v[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const uint32_t jo = of0 + row + 16 * p, ji = if0 + 4 * quad;
    v[p] = u32x4{0, 0, 0, 0};
    if (jo < a.n_out_fast && ji < a.n_in_fast) {
      v[p] = *reinterpret_cast<const u32x4 *>(in + off_in + static_cast<int32_t>(jo) * a.in_stride_of_out_fast +
                                              static_cast<int32_t>(ji));
    }
  }
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    tile[4 * quad + 0][row + 16 * p] = v[p].x;
    tile[4 * quad + 1][row + 16 * p] = v[p].y;
    tile[4 * quad + 2][row + 16 * p] = v[p].z;
    tile[4 * quad + 3][row + 16 * p] = v[p].w;
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const uint32_t ji = if0 + row + 16 * p, jo = of0 + 4 * quad;
    if (jo < a.n_out_fast && ji < a.n_in_fast) {
      const uint32_t *t = &tile[row + 16 * p][4 * quad];
      StoreMaybeStreaming(reinterpret_cast<u32x4 *>(out + off_out + static_cast<int32_t>(ji) * a.out_stride_of_in_fast +
                                                    static_cast<int32_t>(jo)),
                          u32x4{t[0], t[1], t[2], t[3]}, streaming);
    }
  }
}

// Launches the tiled kernel when `nest` (operand 0 = out, 1 = in, 32-bit elements) is a transposing copy of
// useful size; false = use the generic element-per-lane path.
bool TryTiledCopy(LoopNest nest, const fl_tensor *in, const fl_tensor *out, hipStream_t stream) {
  nest.Canonicalise();
  const int inner = nest.rank - 1;
  if (nest.rank < 2 || nest.strides[0][inner] != 1 || nest.strides[1][inner] == 1) return false;
  int in_fast = -1;
  for (int d = 0; d < inner; ++d) {
    if (nest.strides[1][d] == 1) in_fast = d;
  }
  if (in_fast < 0 || nest.shape[inner] < 32 || nest.shape[in_fast] < 32) return false;
  TiledCopyArgs a;
  std::memset(&a, 0, sizeof(a));
  a.n_out_fast = static_cast<uint32_t>(nest.shape[inner]);
  a.n_in_fast = static_cast<uint32_t>(nest.shape[in_fast]);
  a.in_stride_of_out_fast = static_cast<int32_t>(nest.strides[1][inner]);
  a.out_stride_of_in_fast = static_cast<int32_t>(nest.strides[0][in_fast]);
  a.tiles_out_fast = (a.n_out_fast + 63) / 64;
  a.tiles_in_fast = (a.n_in_fast + 63) / 64;
  LoopNest outer;
  outer.n_operands = 2;
  outer.rank = 0;
  int64_t n_outer = 1;
  for (int d = 0; d < inner; ++d) {
    if (d == in_fast) continue;
    outer.shape[outer.rank] = nest.shape[d];
    outer.strides[0][outer.rank] = nest.strides[0][d];
    outer.strides[1][outer.rank] = nest.strides[1][d];
    n_outer *= nest.shape[d];
    ++outer.rank;
  }
  if (outer.rank == 0) {
    outer.rank = 1;
    outer.shape[0] = 1;
  }
  const int64_t blocks = n_outer * a.tiles_out_fast * a.tiles_in_fast;
  if (blocks > INT32_MAX) return false;
  a.outer = MakeNestArgs<2>(outer);
  a.streaming = StreamingOutput(static_cast<size_t>(n_outer) * a.n_out_fast * a.n_in_fast * sizeof(uint32_t)) ? 1 : 0;
  bool vec = a.n_out_fast % 4 == 0 && a.n_in_fast % 4 == 0 && a.in_stride_of_out_fast % 4 == 0 &&
             a.out_stride_of_in_fast % 4 == 0 && IsAligned(in->base, 16) && IsAligned(out->base, 16);
  for (int d = 0; d < outer.rank && vec; ++d) {
    vec = outer.shape[d] == 1 || (outer.strides[0][d] % 4 == 0 && outer.strides[1][d] % 4 == 0);
  }
  if (vec) {
    FL_LAUNCH(TiledCopyVecKernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream, a,
              static_cast<uint32_t *>(out->base), static_cast<const uint32_t *>(in->base));
  } else {
    FL_LAUNCH(TiledCopyKernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream, a,
              static_cast<uint32_t *>(out->base), static_cast<const uint32_t *>(in->base));
  }
  return true;
}

// Copy `in` (already re-strided to the output's index space) into `out`,
// whatever the (equal) element type is.
int CopyNest(const LoopNest &nest, const fl_tensor *in, const fl_tensor *out, void *stream) {
  if (in->dtype != out->dtype) return FL_ERR_DTYPE;
  if (DtypeSize(out->dtype) == 4 && TryTiledCopy(nest, in, out, AsStream(stream))) return LaunchStatus();
  switch (DtypeSize(out->dtype)) {
    case 1: return Unary<uint8_t, uint8_t>(nest, in, out, Copy<uint8_t, uint8_t>{}, stream);
    case 2: return Unary<uint16_t, uint16_t>(nest, in, out, Copy<uint16_t, uint16_t>{}, stream);
    case 4: return Unary<uint32_t, uint32_t>(nest, in, out, Copy<uint32_t, uint32_t>{}, stream);
    case 8: return Unary<uint64_t, uint64_t>(nest, in, out, Copy<uint64_t, uint64_t>{}, stream);
    default: return FL_ERR_DTYPE;
  }
}

}  // namespace

// Shared with other translation units: strided copy of `in` viewed with
// `in_strides`/`in_offset` over the index space `shape` of the output view.
int StridedCopy(const fl_tensor *in, int64_t in_offset, const int64_t *in_strides, const fl_tensor *out,
                int64_t out_offset, int rank, const int64_t *shape, const int64_t *out_strides, void *stream) {
  LoopNest nest;
  nest.rank = rank;
  nest.n_operands = 2;
  for (int i = 0; i < rank; ++i) {
    nest.shape[i] = shape[i];
    nest.strides[0][i] = out_strides[i];
    nest.strides[1][i] = in_strides[i];
  }
  fl_tensor i2 = *in, o2 = *out;
  const size_t esz = DtypeSize(in->dtype);
  i2.base = static_cast<char *>(in->base) + in_offset * static_cast<int64_t>(esz);
  o2.base = static_cast<char *>(out->base) + out_offset * static_cast<int64_t>(esz);
  return CopyNest(nest, &i2, &o2, stream);
}

namespace {

// Elementwise chain on two tensors stored identically (the usual case): flat 128-bit accesses, eight values
// per lane (two quads 256 lanes apart, so that each access of a wave covers one contiguous kilobyte), one
// wave-uniform branch per chain step for all eight.
__global__ __launch_bounds__(256) void ChainFlatKernel(fl_ew_program g, uint32_t n_vec8, float *__restrict__ out,
                                                       const float *__restrict__ in, bool streaming) {
  typedef float float4v __attribute__((ext_vector_type(4)));
  const uint32_t n_vec4 = 2 * n_vec8;
  const uint32_t i0 = blockIdx.x * 512 + threadIdx.x, i1 = i0 + 256;
  if (i0 >= n_vec4) return;
  const bool second = i1 < n_vec4;
  const float4v lo = reinterpret_cast<const float4v *>(in)[i0];
  const float4v hi = second ? reinterpret_cast<const float4v *>(in)[i1] : float4v{1.0f, 1.0f, 1.0f, 1.0f};
  float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  RunChainBlock<8>(g, v);
  StoreMaybeStreaming(reinterpret_cast<float4v *>(out) + i0, float4v{v[0], v[1], v[2], v[3]}, streaming);
  if (second) StoreMaybeStreaming(reinterpret_cast<float4v *>(out) + i1, float4v{v[4], v[5], v[6], v[7]}, streaming);
}

// Pad: one lane per output element; inside the interior it copies the input, outside it writes zero.
struct PadArgs {
  NestArgs<2> nest;  // dims of the OUTPUT in descending output-stride order; operand 1 = input strides
  uint32_t lo[kMaxRank], hi[kMaxRank];
  uint32_t n;
  int32_t in_base;  // sum lo[d] * input stride[d]
};

template <typename T>
__global__ __launch_bounds__(256) void PadKernel(PadArgs p, T *__restrict__ out, const T *__restrict__ in) {
  const uint32_t item = blockIdx.x * 256 + threadIdx.x;
  if (item >= p.n) return;
  uint32_t rem = item;
  int32_t off_out = 0, off_in = 0;
  bool inside = true;
  for (int d = p.nest.rank - 1; d >= 0; --d) {
    uint32_t q = 0, r = rem;
    if (d > 0) p.nest.dims[d].div.DivMod(rem, q, r);
    rem = q;
    off_out += static_cast<int32_t>(r) * p.nest.dims[d].strides[0];
    off_in += static_cast<int32_t>(r) * p.nest.dims[d].strides[1];
    inside = inside && r >= p.lo[d] && r < p.hi[d];
  }
  out[off_out] = inside ? in[off_in - p.in_base] : T(0);
}

template <typename T>
int LaunchPad(const fl_tensor *in, const fl_tensor *out, const int64_t *before, hipStream_t stream) {
  // dims sorted by descending output stride (innermost loop = fastest output dim), nothing merged
  int order[kMaxRank];
  for (int i = 0; i < out->rank; ++i) order[i] = i;
  for (int i = 1; i < out->rank; ++i) {
    for (int j = i; j > 0 && out->strides[order[j]] > out->strides[order[j - 1]]; --j) std::swap(order[j], order[j - 1]);
  }
  LoopNest nest;
  nest.n_operands = 2;
  nest.rank = out->rank;
  PadArgs p;
  std::memset(&p, 0, sizeof(p));
  int64_t total = 1, in_base = 0;
  for (int k = 0; k < out->rank; ++k) {
    const int d = order[k];
    nest.shape[k] = out->shape[d];
    nest.strides[0][k] = out->strides[d];
    nest.strides[1][k] = in->strides[d];
    p.lo[k] = static_cast<uint32_t>(before[d]);
    p.hi[k] = static_cast<uint32_t>(before[d] + in->shape[d]);
    in_base += before[d] * in->strides[d];
    total *= out->shape[d];
  }
  if (total == 0) return FL_OK;
  if (total > 0x7fffffff) return FL_ERR_TOO_LARGE;
  p.nest = MakeNestArgs<2>(nest);
  p.n = static_cast<uint32_t>(total);
  p.in_base = static_cast<int32_t>(in_base);
  FL_LAUNCH(PadKernel<T>, dim3((p.n + 255) / 256), dim3(256), 0, stream, p, static_cast<T *>(out->base),
            static_cast<const T *>(in->base));
  return LaunchStatus();
}

// Rotary position embedding: one lane per output element.  Operands of the nest: 0 = out, 1 = x, 2 = cos, 3 = sin;
// the last nest dim is the rotated axis (kept apart so that its coordinate is at hand).
struct RotaryArgs {
  NestArgs<4> nest;
  uint32_t n;
  uint32_t rot, half;  // the first `rot` values of the axis are rotated, partner at distance half = rot / 2
  int32_t x_half;      // half * (stride of x along the axis)
};

__device__ __forceinline__ void RotaryItem(const RotaryArgs &p, uint32_t item, float *__restrict__ out,
                                           const float *__restrict__ x, const float *__restrict__ cos_t,
                                           const float *__restrict__ sin_t) {
  if (item >= p.n) return;
  uint32_t rem = item, d = 0;
  int32_t off[4] = {0, 0, 0, 0};
  for (int k = p.nest.rank - 1; k >= 0; --k) {
    uint32_t q = 0, r = rem;
    if (k > 0) p.nest.dims[k].div.DivMod(rem, q, r);
    rem = q;
    if (k == p.nest.rank - 1) d = r;
#pragma unroll
    for (int o = 0; o < 4; ++o) off[o] += static_cast<int32_t>(r) * p.nest.dims[k].strides[o];
  }
  float v = x[off[1]];
  if (d < p.rot) {
    // rot = concat(-x[half:rot], x[:half]); each product is rounded before the sum, like the separate kernels
#pragma clang fp contract(off)
    const float partner = d < p.half ? -x[off[1] + p.x_half] : x[off[1] - p.x_half];
    const float direct = v * cos_t[off[2]];
    const float turned = partner * sin_t[off[3]];
    v = direct + turned;
  }
  out[off[0]] = v;
}

__global__ __launch_bounds__(256) void RotaryKernel(RotaryArgs p, float *__restrict__ out, const float *__restrict__ x,
                                                    const float *__restrict__ cos_t, const float *__restrict__ sin_t) {
  RotaryItem(p, blockIdx.x * 256 + threadIdx.x, out, x, cos_t, sin_t);
}

// Two tensors against the same tables in one launch (the queries and the keys of a layer): blockIdx.y picks the problem.
__global__ __launch_bounds__(256) void RotaryPairKernel(RotaryArgs p0, RotaryArgs p1, float *__restrict__ out0,
                                                        const float *__restrict__ x0, float *__restrict__ out1,
                                                        const float *__restrict__ x1, const float *__restrict__ cos_t,
                                                        const float *__restrict__ sin_t) {
  const uint32_t item = blockIdx.x * 256 + threadIdx.x;
  if (blockIdx.y == 0) RotaryItem(p0, item, out0, x0, cos_t, sin_t);
  else RotaryItem(p1, item, out1, x1, cos_t, sin_t);
}

// validates one problem and fills its arguments (n = 0: nothing to do)
int MakeRotaryArgs(const fl_tensor *x, const fl_tensor *cos_t, const fl_tensor *sin_t, const fl_tensor *out,
                   int64_t rotary_dims, RotaryArgs *args) {
  RotaryArgs &p = *args;
  std::memset(&p, 0, sizeof(p));
  FL_CHECK(CheckView(x));
  FL_CHECK(CheckView(cos_t));
  FL_CHECK(CheckView(sin_t));
  FL_CHECK(CheckView(out));
  if (x->dtype != FL_FLOAT32 || cos_t->dtype != FL_FLOAT32 || sin_t->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32)
    return FL_ERR_DTYPE;
  if (!SameShape(x, out)) return FL_ERR_SHAPE;
  const int rank = out->rank;
  if (rank < 1) return FL_ERR_RANK;
  const int64_t len = out->shape[rank - 1];
  if (rotary_dims < 0 || rotary_dims > len || rotary_dims % 2 != 0) return FL_ERR_ATTR;
  LoopNest nest;
  nest.rank = rank;
  nest.n_operands = 4;
  int64_t total = 1;
  for (int i = 0; i < rank; ++i) {
    nest.shape[i] = out->shape[i];
    nest.strides[0][i] = out->strides[i];
    nest.strides[1][i] = x->strides[i];
    total *= out->shape[i];
  }
  // cos and sin: [.., rotary_dims], leading dims broadcast to x's; never read beyond rotary_dims
  const fl_tensor *tables[2] = {cos_t, sin_t};
  for (int k = 0; k < 2; ++k) {
    const fl_tensor *t = tables[k];
    if (t->rank < 1 || t->rank > rank || t->shape[t->rank - 1] != rotary_dims) return FL_ERR_SHAPE;
    for (int i = 0; i < rank; ++i) {
      const int j = t->rank - rank + i;
      if (i == rank - 1) nest.strides[2 + k][i] = t->strides[j];
      else if (j < 0 || t->shape[j] == 1) nest.strides[2 + k][i] = 0;
      else if (t->shape[j] == out->shape[i]) nest.strides[2 + k][i] = t->strides[j];
      else return FL_ERR_SHAPE;
    }
  }
  if (total == 0) return FL_OK;
  if (total > 0x7fffffff) return FL_ERR_TOO_LARGE;
  p.nest = MakeNestArgs<4>(nest);
  p.n = static_cast<uint32_t>(total);
  p.rot = static_cast<uint32_t>(rotary_dims);
  p.half = static_cast<uint32_t>(rotary_dims / 2);
  p.x_half = static_cast<int32_t>((rotary_dims / 2) * x->strides[rank - 1]);
  return FL_OK;
}

int LaunchRotary(const fl_tensor *x, const fl_tensor *cos_t, const fl_tensor *sin_t, const fl_tensor *out,
                 int64_t rotary_dims, hipStream_t stream) {
  RotaryArgs p;
  FL_CHECK(MakeRotaryArgs(x, cos_t, sin_t, out, rotary_dims, &p));
  if (p.n == 0) return FL_OK;
  FL_LAUNCH(RotaryKernel, dim3((p.n + 255) / 256), dim3(256), 0, stream, p, static_cast<float *>(out->base),
            static_cast<const float *>(x->base), static_cast<const float *>(cos_t->base),
            static_cast<const float *>(sin_t->base));
  return LaunchStatus();
}

int LaunchRotaryPair(const fl_tensor *x0, const fl_tensor *out0, const fl_tensor *x1, const fl_tensor *out1,
                     const fl_tensor *cos_t, const fl_tensor *sin_t, int64_t rotary_dims, hipStream_t stream) {
  RotaryArgs p0, p1;
  FL_CHECK(MakeRotaryArgs(x0, cos_t, sin_t, out0, rotary_dims, &p0));
  FL_CHECK(MakeRotaryArgs(x1, cos_t, sin_t, out1, rotary_dims, &p1));
  const uint32_t n = std::max(p0.n, p1.n);
  if (n == 0) return FL_OK;
  FL_LAUNCH(RotaryPairKernel, dim3((n + 255) / 256, 2), dim3(256), 0, stream, p0, p1, static_cast<float *>(out0->base),
            static_cast<const float *>(x0->base), static_cast<float *>(out1->base), static_cast<const float *>(x1->base),
            static_cast<const float *>(cos_t->base), static_cast<const float *>(sin_t->base));
  return LaunchStatus();
}

}  // namespace
}  // namespace fl

using namespace fl;

extern "C" {

int fluidml_hip_add_constant(const fl_tensor *in, const fl_tensor *out, double value, void *stream) {
  LoopNest nest;
  FL_CHECK(IdentityNest(in, out, &nest));
  if (in->dtype != out->dtype) return FL_ERR_DTYPE;
  switch (in->dtype) {
    case FL_FLOAT32: return Unary<float, float>(nest, in, out, AddC<float>{static_cast<float>(value)}, stream);
    case FL_INT32: return Unary<int32_t, int32_t>(nest, in, out, AddC<int32_t>{static_cast<int32_t>(value)}, stream);
    case FL_INT64: return Unary<int64_t, int64_t>(nest, in, out, AddC<int64_t>{static_cast<int64_t>(value)}, stream);
    default: return FL_ERR_DTYPE;
  }
}

int fluidml_hip_add_common(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream) {
  if (!lhs || !rhs || !out) return FL_ERR_NULL;
  if (lhs->dtype != FL_FLOAT32 || rhs->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  return Binary<float>(lhs, rhs, out, Add2<float>{}, stream);
}

int fluidml_hip_mul_add(const fl_tensor *a, const fl_tensor *b, const fl_tensor *c, const fl_tensor *out, void *stream) {
  if (!a || !b || !c || !out) return FL_ERR_NULL;
  if (a->dtype != FL_FLOAT32 || b->dtype != FL_FLOAT32 || c->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  const fl_tensor *ins[3] = {a, b, c};
  LoopNest nest;
  FL_CHECK(BroadcastNest(ins, 3, out, &nest));
  return LaunchNest<3, float, float, float, float>(nest, out->base, a->base, b->base, c->base, MulAdd3{}, AsStream(stream));
}

int fluidml_hip_add_add(const fl_tensor *a, const fl_tensor *b, const fl_tensor *c, const fl_tensor *out, void *stream) {
  if (!a || !b || !c || !out) return FL_ERR_NULL;
  if (a->dtype != FL_FLOAT32 || b->dtype != FL_FLOAT32 || c->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  const fl_tensor *ins[3] = {a, b, c};
  LoopNest nest;
  FL_CHECK(BroadcastNest(ins, 3, out, &nest));
  return LaunchNest<3, float, float, float, float>(nest, out->base, a->base, b->base, c->base, AddAdd3{}, AsStream(stream));
}

int fluidml_hip_rotary(const fl_tensor *x, const fl_tensor *cos_table, const fl_tensor *sin_table, const fl_tensor *out,
                       int64_t rotary_dims, void *stream) {
  if (!x || !cos_table || !sin_table || !out) return FL_ERR_NULL;
  return LaunchRotary(x, cos_table, sin_table, out, rotary_dims, AsStream(stream));
}

int fluidml_hip_rotary_pair(const fl_tensor *x0, const fl_tensor *out0, const fl_tensor *x1, const fl_tensor *out1,
                            const fl_tensor *cos_table, const fl_tensor *sin_table, int64_t rotary_dims, void *stream) {
  if (!x0 || !out0 || !x1 || !out1 || !cos_table || !sin_table) return FL_ERR_NULL;
  return LaunchRotaryPair(x0, out0, x1, out1, cos_table, sin_table, rotary_dims, AsStream(stream));
}

int fluidml_hip_sub_constant_lhs(const fl_tensor *in, const fl_tensor *out, double value, void *stream) {
  return UnaryF32(in, out, RSubC<float>{static_cast<float>(value)}, stream);
}

int fluidml_hip_sub_common(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream) {
  if (!lhs || !rhs || !out) return FL_ERR_NULL;
  if (lhs->dtype != FL_FLOAT32 || rhs->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  return Binary<float>(lhs, rhs, out, Sub2<float>{}, stream);
}

int fluidml_hip_mul_constant(const fl_tensor *in, const fl_tensor *out, double value, void *stream) {
  return UnaryF32(in, out, MulC<float>{static_cast<float>(value)}, stream);
}

int fluidml_hip_mul_common(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream) {
  if (!lhs || !rhs || !out) return FL_ERR_NULL;
  if (lhs->dtype != rhs->dtype || lhs->dtype != out->dtype) return FL_ERR_DTYPE;
  switch (out->dtype) {
    case FL_FLOAT32: return Binary<float>(lhs, rhs, out, Mul2<float>{}, stream);
    case FL_INT32: return Binary<int32_t>(lhs, rhs, out, Mul2<int32_t>{}, stream);
    case FL_INT64: return Binary<int64_t>(lhs, rhs, out, Mul2<int64_t>{}, stream);
    default: return FL_ERR_DTYPE;
  }
}

int fluidml_hip_div_constant_rhs(const fl_tensor *in, const fl_tensor *out, double value, void *stream) {
  return UnaryF32(in, out, DivC{static_cast<float>(value)}, stream);
}

int fluidml_hip_div_common(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream) {
  if (!lhs || !rhs || !out) return FL_ERR_NULL;
  if (lhs->dtype != FL_FLOAT32 || rhs->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  return Binary<float>(lhs, rhs, out, Div2{}, stream);
}

int fluidml_hip_pow(const fl_tensor *in, const fl_tensor *out, double exponent, void *stream) {
  return UnaryF32(in, out, PowC{static_cast<float>(exponent)}, stream);
}

int fluidml_hip_erf(const fl_tensor *in, const fl_tensor *out, void *stream) { return UnaryF32(in, out, Erf{}, stream); }

int fluidml_hip_relu(const fl_tensor *in, const fl_tensor *out, void *stream) { return UnaryF32(in, out, Relu{}, stream); }

int fluidml_hip_clip(const fl_tensor *in, const fl_tensor *out, float lo, float hi, void *stream) {
  return UnaryF32(in, out, Clip{lo, hi}, stream);
}

int fluidml_hip_tanh(const fl_tensor *in, const fl_tensor *out, void *stream) { return UnaryF32(in, out, Tanh{}, stream); }

int fluidml_hip_sqrt(const fl_tensor *in, const fl_tensor *out, void *stream) { return UnaryF32(in, out, Sqrt{}, stream); }

int fluidml_hip_neg(const fl_tensor *in, const fl_tensor *out, void *stream) { return UnaryF32(in, out, Neg{}, stream); }

int fluidml_hip_not(const fl_tensor *in, const fl_tensor *out, void *stream) {
  LoopNest nest;
  FL_CHECK(IdentityNest(in, out, &nest));
  if (in->dtype != FL_BOOL || out->dtype != FL_BOOL) return FL_ERR_DTYPE;
  return Unary<uint8_t, uint8_t>(nest, in, out, Not{}, stream);
}

int fluidml_hip_cast(const fl_tensor *in, const fl_tensor *out, void *stream) {
  LoopNest nest;
  FL_CHECK(IdentityNest(in, out, &nest));
#define FL_CAST_CASE(TI_E, TI, TO_E, TO) \
  if (in->dtype == TI_E && out->dtype == TO_E) return Unary<TO, TI>(nest, in, out, Copy<TO, TI>{}, stream)
  FL_CAST_CASE(FL_BOOL, uint8_t, FL_BOOL, uint8_t);
  FL_CAST_CASE(FL_BOOL, uint8_t, FL_INT32, int32_t);
  FL_CAST_CASE(FL_BOOL, uint8_t, FL_INT64, int64_t);
  FL_CAST_CASE(FL_INT32, int32_t, FL_INT32, int32_t);
  FL_CAST_CASE(FL_INT32, int32_t, FL_INT64, int64_t);
  FL_CAST_CASE(FL_INT64, int64_t, FL_INT32, int32_t);
  FL_CAST_CASE(FL_INT64, int64_t, FL_INT64, int64_t);
#undef FL_CAST_CASE
  return FL_ERR_DTYPE;
}

int fluidml_hip_equal(const fl_tensor *in, const fl_tensor *out, double value, void *stream) {
  LoopNest nest;
  FL_CHECK(IdentityNest(in, out, &nest));
  if (in->dtype != FL_INT64 || out->dtype != FL_BOOL) return FL_ERR_DTYPE;
  return Unary<uint8_t, int64_t>(nest, in, out, EqC{static_cast<int64_t>(value)}, stream);
}

int fluidml_hip_dropout(const fl_tensor *in, const fl_tensor *out, void *stream) {
  LoopNest nest;
  FL_CHECK(IdentityNest(in, out, &nest));
  return CopyNest(nest, in, out, stream);
}

int fluidml_hip_where_constant_cond_constant_scalar_y(const fl_tensor *cond, const fl_tensor *x, const fl_tensor *out,
                                                      double y, void *stream) {
  if (!cond || !x || !out) return FL_ERR_NULL;
  if (cond->dtype != FL_BOOL || x->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  const fl_tensor *ins[2] = {cond, x};
  LoopNest nest;
  FL_CHECK(BroadcastNest(ins, 2, out, &nest));
  return LaunchNest<2, float, uint8_t, float, Empty>(nest, out->base, cond->base, x->base, nullptr,
                                                     WhereScalarY{static_cast<float>(y)}, AsStream(stream));
}

int fluidml_hip_where_constant_cond_constant_tensor_y(const fl_tensor *cond, const fl_tensor *x, const fl_tensor *y,
                                                      const fl_tensor *out, void *stream) {
  if (!cond || !x || !y || !out) return FL_ERR_NULL;
  if (cond->dtype != FL_BOOL || x->dtype != FL_FLOAT32 || y->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32)
    return FL_ERR_DTYPE;
  const fl_tensor *ins[3] = {cond, x, y};
  LoopNest nest;
  FL_CHECK(BroadcastNest(ins, 3, out, &nest));
  return LaunchNest<3, float, uint8_t, float, float>(nest, out->base, cond->base, x->base, y->base, WhereTensorY{},
                                                     AsStream(stream));
}

int fluidml_hip_add_div_erf_add_mul_mul(const fl_tensor *in, const fl_tensor *add0, const fl_tensor *out, double div,
                                        double add1, double mul1, void *stream) {
  if (!in || !add0 || !out) return FL_ERR_NULL;
  if (in->dtype != FL_FLOAT32 || add0->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  const fl_tensor *ins[2] = {in, add0};
  LoopNest nest;
  FL_CHECK(BroadcastNest(ins, 2, out, &nest));
  return LaunchNest<2, float, float, float, Empty>(
      nest, out->base, in->base, add0->base, nullptr,
      Gelu{static_cast<float>(div), static_cast<float>(add1), static_cast<float>(mul1)}, AsStream(stream));
}

// Strides of `in` in the index space of an output that has extra unit dims at
// `axes` (negative axes count from the output rank).
static int UnsqueezedStrides(const fl_tensor *in, const fl_tensor *out, const int64_t *axes, int32_t n_axes,
                             int64_t *strides) {
  if (n_axes < 0 || (n_axes > 0 && axes == nullptr)) return FL_ERR_ATTR;
  if (in->rank + n_axes != out->rank) return FL_ERR_RANK;
  int j = 0;
  for (int i = 0; i < out->rank; ++i) {
    bool is_axis = false;
    for (int k = 0; k < n_axes; ++k) {
      const int64_t ax = axes[k] < 0 ? axes[k] + out->rank : axes[k];
      if (ax < 0 || ax >= out->rank) return FL_ERR_ATTR;
      if (ax == i) is_axis = true;
    }
    if (is_axis) {
      if (out->shape[i] != 1) return FL_ERR_SHAPE;
      strides[i] = 0;
    } else {
      if (j >= in->rank || in->shape[j] != out->shape[i]) return FL_ERR_SHAPE;
      strides[i] = in->strides[j++];
    }
  }
  return j == in->rank ? FL_OK : FL_ERR_SHAPE;
}

int fluidml_hip_unsqueeze_sub_lhs_scalar_mul_rhs_scalar(const fl_tensor *in, const fl_tensor *out, const int64_t *axes,
                                                        int32_t n_axes, double sub, double mul, void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (in->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  LoopNest nest;
  nest.rank = out->rank;
  nest.n_operands = 2;
  FL_CHECK(UnsqueezedStrides(in, out, axes, n_axes, nest.strides[1]));
  for (int i = 0; i < out->rank; ++i) {
    nest.shape[i] = out->shape[i];
    nest.strides[0][i] = out->strides[i];
  }
  return Unary<float, float>(nest, in, out, SubMul{static_cast<float>(sub), static_cast<float>(mul)}, stream);
}

int fluidml_hip_unsqueeze(const fl_tensor *in, const fl_tensor *out, const int64_t *axes, int32_t n_axes, void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  LoopNest nest;
  nest.rank = out->rank;
  nest.n_operands = 2;
  FL_CHECK(UnsqueezedStrides(in, out, axes, n_axes, nest.strides[1]));
  for (int i = 0; i < out->rank; ++i) {
    nest.shape[i] = out->shape[i];
    nest.strides[0][i] = out->strides[i];
  }
  return CopyNest(nest, in, out, stream);
}

int fluidml_hip_squeeze(const fl_tensor *in, const fl_tensor *out, const int64_t *axes, int32_t n_axes, void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (n_axes < 0 || (n_axes > 0 && axes == nullptr)) return FL_ERR_ATTR;
  if (in->rank != out->rank + n_axes) return FL_ERR_RANK;
  // reference squeeze.cpp:17-54 matches axes against the raw input index
  LoopNest nest;
  nest.rank = out->rank;
  nest.n_operands = 2;
  int j = 0;
  for (int i = 0; i < in->rank; ++i) {
    bool squeezed = false;
    for (int k = 0; k < n_axes; ++k) {
      const int64_t ax = axes[k] < 0 ? axes[k] + in->rank : axes[k];
      if (ax == i) squeezed = true;
    }
    if (squeezed) {
      if (in->shape[i] != 1) return FL_ERR_SHAPE;
    } else {
      if (j >= out->rank || out->shape[j] != in->shape[i]) return FL_ERR_SHAPE;
      nest.shape[j] = out->shape[j];
      nest.strides[0][j] = out->strides[j];
      nest.strides[1][j] = in->strides[i];
      ++j;
    }
  }
  if (j != out->rank) return FL_ERR_SHAPE;
  return CopyNest(nest, in, out, stream);
}

int fluidml_hip_transpose(const fl_tensor *in, const fl_tensor *out, const int64_t *perm, int32_t n_perm, void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (perm == nullptr) return FL_ERR_NULL;
  if (n_perm != in->rank || in->rank != out->rank) return FL_ERR_RANK;
  LoopNest nest;
  nest.rank = out->rank;
  nest.n_operands = 2;
  bool seen[kMaxRank] = {};
  for (int i = 0; i < out->rank; ++i) {
    const int64_t p = perm[i];
    if (p < 0 || p >= in->rank || seen[p]) return FL_ERR_ATTR;
    seen[p] = true;
    if (out->shape[i] != in->shape[p]) return FL_ERR_SHAPE;
    nest.shape[i] = out->shape[i];
    nest.strides[0][i] = out->strides[i];
    nest.strides[1][i] = in->strides[p];
  }
  return CopyNest(nest, in, out, stream);
}

int fluidml_hip_slice(const fl_tensor *in, const fl_tensor *out, const int64_t *starts, const int64_t *axes,
                      const int64_t *steps, int32_t n, void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (in->rank != out->rank) return FL_ERR_RANK;
  if (n < 0 || (n > 0 && (!starts || !axes || !steps))) return FL_ERR_ATTR;
  int64_t offs[kMaxRank] = {}, step[kMaxRank];
  for (int i = 0; i < in->rank; ++i) step[i] = 1;
  for (int k = 0; k < n; ++k) {
    const int64_t ax = axes[k];
    if (ax < 0 || ax >= in->rank || steps[k] <= 0 || starts[k] < 0) return FL_ERR_ATTR;
    offs[ax] = starts[k];
    step[ax] = steps[k];
  }
  int64_t in_offset = 0, in_strides[kMaxRank];
  for (int i = 0; i < in->rank; ++i) {
    if (offs[i] + (out->shape[i] - 1) * step[i] >= in->shape[i]) return FL_ERR_SHAPE;
    in_offset += offs[i] * in->strides[i];
    in_strides[i] = in->strides[i] * step[i];
  }
  return StridedCopy(in, in_offset, in_strides, out, 0, out->rank, out->shape, out->strides, stream);
}

int fluidml_hip_concat2(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, int64_t axis, void *stream) {
  FL_CHECK(CheckView(lhs));
  FL_CHECK(CheckView(rhs));
  FL_CHECK(CheckView(out));
  if (lhs->rank != out->rank || rhs->rank != out->rank) return FL_ERR_RANK;
  if (axis < 0 || axis >= out->rank) return FL_ERR_ATTR;
  if (lhs->dtype != out->dtype || rhs->dtype != out->dtype) return FL_ERR_DTYPE;
  for (int i = 0; i < out->rank; ++i) {
    if (i == axis) {
      if (lhs->shape[i] + rhs->shape[i] != out->shape[i]) return FL_ERR_SHAPE;
    } else if (lhs->shape[i] != out->shape[i] || rhs->shape[i] != out->shape[i]) {
      return FL_ERR_SHAPE;
    }
  }
  FL_CHECK(StridedCopy(lhs, 0, lhs->strides, out, 0, out->rank, lhs->shape, out->strides, stream));
  return StridedCopy(rhs, 0, rhs->strides, out, lhs->shape[axis] * out->strides[axis], out->rank, rhs->shape,
                     out->strides, stream);
}

int fluidml_hip_elementwise_chain(const fl_tensor *in, const fl_tensor *out, const fl_ew_program *chain, void *stream) {
  if (chain == nullptr) return FL_ERR_NULL;
  FL_CHECK(CheckChain(chain));
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (in->dtype == FL_FLOAT32 && out->dtype == FL_FLOAT32 && SameShape(in, out)) {
    // same dense storage on both sides?
    bool same = true;
    int64_t numel = 1, span = 0;
    for (int i = 0; i < in->rank; ++i) {
      same = same && (in->strides[i] == out->strides[i] || in->shape[i] == 1);
      numel *= in->shape[i];
      span += (in->shape[i] - 1) * in->strides[i];
    }
    if (same && span + 1 == numel && numel % 8 == 0 && IsAligned(in->base, 16) && IsAligned(out->base, 16)) {
      const uint32_t n_vec8 = static_cast<uint32_t>(numel / 8);
      FL_LAUNCH(ChainFlatKernel, dim3((n_vec8 + 255) / 256), dim3(256), 0, AsStream(stream), *chain, n_vec8,
                static_cast<float *>(out->base), static_cast<const float *>(in->base),
                StreamingOutput(static_cast<size_t>(numel) * sizeof(float)));
      return LaunchStatus();
    }
  }
  return UnaryF32(in, out, Chain{*chain}, stream);
}

int fluidml_hip_pad(const fl_tensor *in, const fl_tensor *out, const int64_t *pads_before, int32_t n, uint32_t flags,
                    void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (in->rank != out->rank || n != in->rank) return FL_ERR_RANK;
  if (in->dtype != out->dtype) return FL_ERR_DTYPE;
  if (pads_before == nullptr && n > 0) return FL_ERR_NULL;
  int64_t out_offset = 0;
  for (int i = 0; i < in->rank; ++i) {
    if (pads_before[i] < 0 || pads_before[i] + in->shape[i] > out->shape[i]) return FL_ERR_SHAPE;
    out_offset += pads_before[i] * out->strides[i];
  }
  if (flags & FL_REF_PAD_BORDER_UNWRITTEN) {
    return StridedCopy(in, 0, in->strides, out, out_offset, in->rank, in->shape, out->strides, stream);
  }
  switch (DtypeSize(in->dtype)) {
    case 1: return LaunchPad<uint8_t>(in, out, pads_before, AsStream(stream));
    case 4: return LaunchPad<uint32_t>(in, out, pads_before, AsStream(stream));
    case 8: return LaunchPad<uint64_t>(in, out, pads_before, AsStream(stream));
    default: return FL_ERR_DTYPE;
  }
}

int fluidml_hip_gather_constant_index_scalar(const fl_tensor *in, const fl_tensor *out, int64_t axis, int64_t index,
                                             uint32_t flags, void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (in->rank != out->rank + 1) return FL_ERR_RANK;
  // The reference normalises `axis` into a local it never uses and compares
  // loop positions with the raw attribute (gather.cpp:113-124).
  int64_t ax = axis;
  if (!(flags & FL_REF_GATHER_RAW_AXIS) && ax < 0) ax += in->rank;
  if (ax < 0 || ax >= in->rank) return (flags & FL_REF_GATHER_RAW_AXIS) ? FL_ERR_UNSUPPORTED : FL_ERR_ATTR;
  if (index < 0 || index >= in->shape[ax]) return FL_ERR_ATTR;
  int64_t in_strides[kMaxRank];
  for (int i = 0, j = 0; i < in->rank; ++i) {
    if (i == ax) continue;
    if (in->shape[i] != out->shape[j]) return FL_ERR_SHAPE;
    in_strides[j++] = in->strides[i];
  }
  return StridedCopy(in, index * in->strides[ax], in_strides, out, 0, out->rank, out->shape, out->strides, stream);
}

}  // extern "C"
