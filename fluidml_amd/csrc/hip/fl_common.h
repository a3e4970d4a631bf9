// Shared host/device helpers for the gfx950 kernels behind include/fluidml_hip.h.
//
// Every kernel in this backend takes strided views (reference kernels read
// shape and strides from the memref type, src/worker/builder.cpp:234-270), so
// the common work is: validate views on the host, put the loop nest in the
// output's physical order, merge dimensions that are contiguous for every
// operand, and hand the device a small by-value descriptor with 32-bit
// division constants.
#ifndef FLUIDML_AMD_CSRC_HIP_FL_COMMON_H_
#define FLUIDML_AMD_CSRC_HIP_FL_COMMON_H_

#include <utility>

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <cstdint>
#include <cstring>

#include "fluidml_hip.h"

namespace fl {

constexpr int kMaxRank = FL_MAX_RANK;
constexpr int kWave = 64;  // CDNA wavefront

#define FL_HIP_CHECK(expr)                      \
  do {                                          \
    hipError_t fl_err__ = (expr);               \
    if (fl_err__ != hipSuccess) {               \
      return static_cast<int>(fl_err__);        \
    }                                           \
  } while (0)

#define FL_CHECK(expr)            \
  do {                            \
    int fl_rc__ = (expr);         \
    if (fl_rc__ != FL_OK) {       \
      return fl_rc__;             \
    }                             \
  } while (0)

inline hipStream_t AsStream(void *stream) { return static_cast<hipStream_t>(stream); }

// Kernel-exact timing: while a thread has a pair of events installed, every kernel it launches through
// FL_LAUNCH updates them with the dispatch's own begin/end timestamps (hipExtLaunchKernelGGL), which
// excludes launch latency and queue gaps -- the same interval a profiler reports for the kernel.
struct KernelTimer {
  hipEvent_t start = nullptr, stop = nullptr;
};
KernelTimer &ThreadKernelTimer();  // runtime.hip

// First error of this thread's kernel launches since the last LaunchStatus().  The runtime's own "last error" is
// shared with every other user of the runtime in the process (a failed probe inside another library stays there
// until someone reads it), so FL_LAUNCH discards what it finds before the launch and keeps what the launch leaves.
inline thread_local hipError_t t_launch_error = hipSuccess;

#define FL_LAUNCH(kernel, grid, block, shmem, stream, ...)                                                       \
  do {                                                                                                           \
    const ::fl::KernelTimer &fl_timer_ = ::fl::ThreadKernelTimer();                                              \
    (void)hipGetLastError();                                                                                     \
    if (fl_timer_.start != nullptr) {                                                                            \
      hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, fl_timer_.start, fl_timer_.stop, 0, __VA_ARGS__); \
    } else {                                                                                                     \
      hipLaunchKernelGGL(kernel, grid, block, shmem, stream, __VA_ARGS__);                                       \
    }                                                                                                            \
    const hipError_t fl_launch_err_ = hipGetLastError();                                                         \
    if (fl_launch_err_ != hipSuccess && ::fl::t_launch_error == hipSuccess) ::fl::t_launch_error = fl_launch_err_; \
  } while (0)

// Per-stream device memory for kernels that combine partial results across workgroups (split-K
// contractions): 4096 partial 32x32 tiles (16 MiB) and as many arrival counters (zero between launches).
// Launches on one stream run in order, so they can share it; two streams never share.
struct StreamWorkspace {
  float *partials = nullptr;
  uint32_t *counters = nullptr;
};
constexpr size_t kWorkspaceTiles = 4096;
constexpr size_t kWorkspaceTileFloats = 1024;
// The stream's workspace, created on first use.  nullptr when it does not exist yet and cannot be created
// now (the stream is being captured into a graph) or the allocation fails; callers then do without.
StreamWorkspace *GetStreamWorkspace(hipStream_t stream);  // runtime.hip
void DropStreamWorkspace(hipStream_t stream);
// Device address of the current device's fixed split-K scratch (fluidml_hip_matmul_no_alloc), looked up on
// the first call per device; `ptr` may be null.  matmul.hip
int StaticScratch(void **ptr);

// Operands a fused convolution launch may carry besides the reference kernel's own (both optional).
struct ConvExtras {
  // multiplier of the input, one value per channel ([1, C, 1, ..]: the MulCommon of a squeeze-and-excitation block in
  // front of a pointwise convolution); each product is rounded like the separate kernel's
  const fl_tensor *channel_scale = nullptr;
  // tensor of the output's shape and strides, added after the elementwise chain (a residual AddCommon behind it)
  const fl_tensor *addend = nullptr;
  // ... or multiplied with the value instead (a MulCommon behind the convolution)
  bool addend_is_factor = false;
  // second output: the mean of the result over its spatial dims, [N, F, 1, ..] (a ReduceMean behind the convolution)
  const fl_tensor *mean_out = nullptr;
};

// Compile-time loop: body(std::integral_constant<int, 0>) ... body(std::integral_constant<int, N - 1>).
// Unlike `#pragma unroll` it cannot be left rolled, so register arrays indexed by the counter stay in registers.
template <int N, typename F, int... I>
__host__ __device__ __forceinline__ void StaticForImpl(F &&body, std::integer_sequence<int, I...>) {
  (body(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__host__ __device__ __forceinline__ void StaticFor(F &&body) {
  StaticForImpl<N>(static_cast<F &&>(body), std::make_integer_sequence<int, N>{});
}

// Interpreter of fl_ew_program, shared by the elementwise-chain kernel and the contraction epilogues.
// Each case is the expression the standalone kernel of that operation evaluates.
__device__ __forceinline__ float RunChain(const fl_ew_program &g, float x) {
  float v = x;
  for (int i = 0; i < g.n; ++i) {
    const float c = g.c[i];
    switch (g.op[i]) {
      case FL_EW_ADD_C: v = v + c; break;
      case FL_EW_RSUB_C: v = c - v; break;
      case FL_EW_MUL_C: v = v * c; break;
      case FL_EW_DIV_C: v = v / c; break;
      case FL_EW_POW_C: v = powf(v, c); break;
      case FL_EW_ERF: v = erff(v); break;
      case FL_EW_RELU: v = v != v ? v : fmaxf(v, 0.0f); break;
      case FL_EW_TANH: v = tanhf(v); break;
      case FL_EW_SQRT: v = sqrtf(v); break;
      case FL_EW_NEG: v = -v; break;
      case FL_EW_ADD_X: v = v + x; break;
      case FL_EW_MUL_X: v = v * x; break;
      case FL_EW_SUB_X: v = v - x; break;
      case FL_EW_RSUB_X: v = x - v; break;
      case FL_EW_DIV_X: v = v / x; break;
      case FL_EW_RDIV_X: v = x / v; break;
      default: break;
    }
  }
  return v;
}

// The same interpreter over a block of N values held in registers: one (wave-uniform) branch per chain
// step instead of one per value.  `v` holds the chain inputs on entry and the results on exit.
template <int N>
__device__ __forceinline__ void RunChainBlock(const fl_ew_program &g, float (&v)[N]) {
  float x[N];
#pragma unroll
  for (int e = 0; e < N; ++e) x[e] = v[e];
  for (int i = 0; i < g.n; ++i) {
    const float c = g.c[i];
#define FL_EW_CASE(OP, EXPR)               \
  case OP:                                 \
    _Pragma("unroll") for (int e = 0; e < N; ++e) v[e] = (EXPR); \
    break;
    switch (g.op[i]) {
      FL_EW_CASE(FL_EW_ADD_C, v[e] + c)
      FL_EW_CASE(FL_EW_RSUB_C, c - v[e])
      FL_EW_CASE(FL_EW_MUL_C, v[e] * c)
      FL_EW_CASE(FL_EW_DIV_C, v[e] / c)
      FL_EW_CASE(FL_EW_POW_C, powf(v[e], c))
      FL_EW_CASE(FL_EW_ERF, erff(v[e]))
      FL_EW_CASE(FL_EW_RELU, v[e] != v[e] ? v[e] : fmaxf(v[e], 0.0f))
      FL_EW_CASE(FL_EW_TANH, tanhf(v[e]))
      FL_EW_CASE(FL_EW_SQRT, sqrtf(v[e]))
      FL_EW_CASE(FL_EW_NEG, -v[e])
      FL_EW_CASE(FL_EW_ADD_X, v[e] + x[e])
      FL_EW_CASE(FL_EW_MUL_X, v[e] * x[e])
      FL_EW_CASE(FL_EW_SUB_X, v[e] - x[e])
      FL_EW_CASE(FL_EW_RSUB_X, x[e] - v[e])
      FL_EW_CASE(FL_EW_DIV_X, v[e] / x[e])
      FL_EW_CASE(FL_EW_RDIV_X, x[e] / v[e])
      default: break;
    }
#undef FL_EW_CASE
  }
}

inline int CheckChain(const fl_ew_program *g) {
  if (g == nullptr) return FL_OK;
  if (g->n < 0 || g->n > FL_EW_MAX_STEPS) return FL_ERR_ATTR;
  for (int i = 0; i < g->n; ++i) {
    if (g->op[i] < FL_EW_ADD_C || g->op[i] > FL_EW_RDIV_X) return FL_ERR_ATTR;
  }
  return FL_OK;
}

inline int LaunchStatus() {
  const hipError_t err = t_launch_error;
  t_launch_error = hipSuccess;
  return err == hipSuccess ? FL_OK : static_cast<int>(err);
}

inline size_t DtypeSize(int32_t dtype) {
  switch (dtype) {
    case FL_BOOL: return 1;
    case FL_INT32: return 4;
    case FL_INT64: return 8;
    case FL_FLOAT16: return 2;
    case FL_FLOAT32: return 4;
    case FL_FLOAT64: return 8;
    default: return 0;
  }
}

// Division by a run-time constant for dividends below 2^31: one mul-hi and a
// shift on the device instead of a ~40 instruction udiv sequence.
struct FastDiv {
  uint32_t divisor;
  uint32_t multiplier;
  uint32_t shift;

  FastDiv() : divisor(1), multiplier(0), shift(0) {}
  explicit FastDiv(uint32_t d) : divisor(d), multiplier(0), shift(0) {
    if (d > 1) {
      uint32_t log2_ceil = 0;
      while ((1ull << log2_ceil) < d) ++log2_ceil;
      const uint32_t p = 31 + log2_ceil;
      multiplier = static_cast<uint32_t>(((1ull << p) + d - 1) / d);
      shift = p - 32;
    }
  }
  __host__ __device__ __forceinline__ uint32_t Div(uint32_t n) const {
#if defined(__HIP_DEVICE_COMPILE__)
    return divisor == 1 ? n : (__umulhi(n, multiplier) >> shift);
#else
    return n / divisor;
#endif
  }
  __host__ __device__ __forceinline__ void DivMod(uint32_t n, uint32_t &q, uint32_t &r) const {
    q = Div(n);
    r = n - q * divisor;
  }
};

// ---- host-side view checks ------------------------------------------------

inline int CheckView(const fl_tensor *t) {
  if (t == nullptr || t->base == nullptr) return FL_ERR_NULL;
  if (t->rank < 0 || t->rank > kMaxRank) return FL_ERR_RANK;
  if (DtypeSize(t->dtype) == 0) return FL_ERR_DTYPE;
  int64_t numel = 1, span = 0;
  for (int i = 0; i < t->rank; ++i) {
    if (t->shape[i] <= 0) return FL_ERR_SHAPE;
    if (t->strides[i] < 0) return FL_ERR_SHAPE;
    numel *= t->shape[i];
    span += (t->shape[i] - 1) * t->strides[i];
    if (numel > INT32_MAX || span > INT32_MAX) return FL_ERR_TOO_LARGE;
  }
  return FL_OK;
}

inline int64_t Numel(const fl_tensor *t) {
  int64_t n = 1;
  for (int i = 0; i < t->rank; ++i) n *= t->shape[i];
  return n;
}

inline bool SameShape(const fl_tensor *a, const fl_tensor *b) {
  if (a->rank != b->rank) return false;
  for (int i = 0; i < a->rank; ++i) {
    if (a->shape[i] != b->shape[i]) return false;
  }
  return true;
}

inline bool IsAligned(const void *p, size_t bytes) {
  return (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
}

// Outputs this large do not stay in the last-level cache until their reader runs; writing them with
// non-temporal stores keeps them from evicting the data the kernel is still reading.  Measured on a 256 MiB
// copy: 5.5 -> 7.0 TB/s; no difference at 64 MiB and below; non-temporal LOADS were slower at every size.
constexpr size_t kStreamingBytes = size_t{64} << 20;
inline bool StreamingOutput(size_t out_bytes) { return out_bytes >= kStreamingBytes; }

// *p = v with a non-temporal store.  V: any trivially copyable type of 4, 8, 16 or 32 bytes aligned to its
// size; other sizes are stored normally.
template <typename V>
__device__ __forceinline__ void StoreStreaming(V *p, const V &v) {
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  if constexpr (sizeof(V) == 4) {
    __builtin_nontemporal_store(__builtin_bit_cast(uint32_t, v), reinterpret_cast<uint32_t *>(p));
  } else if constexpr (sizeof(V) == 8) {
    __builtin_nontemporal_store(__builtin_bit_cast(u32x2, v), reinterpret_cast<u32x2 *>(p));
  } else if constexpr (sizeof(V) == 16) {
    __builtin_nontemporal_store(__builtin_bit_cast(u32x4, v), reinterpret_cast<u32x4 *>(p));
  } else if constexpr (sizeof(V) == 32) {
    struct Halves {
      u32x4 lo, hi;
    };
    const Halves h = __builtin_bit_cast(Halves, v);
    __builtin_nontemporal_store(h.lo, reinterpret_cast<u32x4 *>(p));
    __builtin_nontemporal_store(h.hi, reinterpret_cast<u32x4 *>(p) + 1);
  } else {
    *p = v;
  }
}

// *p = v, non-temporal when `streaming` (wave-uniform).
template <typename V>
__device__ __forceinline__ void StoreMaybeStreaming(V *p, const V &v, bool streaming) {
  if (!streaming) {
    *p = v;
    return;
  }
  // The two empty statements (which name the address, so that the store cannot move across them even when the
  // pointer is `__restrict__`) keep the optimiser from folding this store and the plain one above into a single
  // store, which would silently lose the non-temporal hint (the merged store keeps only what both had).
  asm volatile("" : : "v"(p) : "memory");
  StoreStreaming(p, v);
  asm volatile("" : : "v"(p) : "memory");
}

// A loop nest over up to kMaxRank dimensions and up to kMaxOperands strided
// operands; operand 0 is the output.  Built in logical order, then
// canonicalised: unit dims dropped, dims ordered by descending output stride
// (so the innermost loop walks the output's fastest physical dimension), and
// neighbours merged when every operand agrees they are contiguous.
constexpr int kMaxOperands = 6;

struct LoopNest {
  int rank = 0;
  int n_operands = 0;
  int64_t shape[kMaxRank] = {};
  int64_t strides[kMaxOperands][kMaxRank] = {};

  void Canonicalise() {
    // drop unit dims
    int w = 0;
    for (int i = 0; i < rank; ++i) {
      if (shape[i] != 1) {
        shape[w] = shape[i];
        for (int o = 0; o < n_operands; ++o) strides[o][w] = strides[o][i];
        ++w;
      }
    }
    rank = w;
    // stable insertion sort by descending output stride; ties keep logical order
    for (int i = 1; i < rank; ++i) {
      for (int j = i; j > 0 && strides[0][j - 1] < strides[0][j]; --j) {
        std::swap(shape[j - 1], shape[j]);
        for (int o = 0; o < n_operands; ++o) std::swap(strides[o][j - 1], strides[o][j]);
      }
    }
    // merge dim i into i-1 when stride[i-1] == stride[i] * shape[i] for all operands
    w = 0;
    for (int i = 0; i < rank; ++i) {
      bool merge = w > 0;
      if (merge) {
        for (int o = 0; o < n_operands; ++o) {
          if (strides[o][w - 1] != strides[o][i] * shape[i]) {
            merge = false;
            break;
          }
        }
      }
      if (merge) {
        shape[w - 1] *= shape[i];
        for (int o = 0; o < n_operands; ++o) strides[o][w - 1] = strides[o][i];
      } else {
        shape[w] = shape[i];
        for (int o = 0; o < n_operands; ++o) strides[o][w] = strides[o][i];
        ++w;
      }
    }
    rank = w;
    if (rank == 0) {
      rank = 1;
      shape[0] = 1;
      for (int o = 0; o < n_operands; ++o) strides[o][0] = 0;
    }
  }
};

// Strides of `t` broadcast against an output of rank `out_rank`/`out_shape`
// with trailing alignment: equal dim -> its stride, dim 1 -> 0 (reference
// GetBroadcastAffineMaps, src/structure/kernel/kernel/utils.cpp:16-52).
inline int BroadcastStrides(const fl_tensor *t, int out_rank, const int64_t *out_shape, int64_t *strides) {
  if (t->rank > out_rank) return FL_ERR_RANK;
  for (int i = 0; i < out_rank; ++i) {
    const int j = t->rank - out_rank + i;
    if (j < 0) {
      strides[i] = 0;
    } else if (t->shape[j] == out_shape[i]) {
      strides[i] = t->strides[j];
    } else if (t->shape[j] == 1) {
      strides[i] = 0;
    } else {
      return FL_ERR_SHAPE;
    }
  }
  return FL_OK;
}

// Device-side descriptor of a canonical loop nest.
#if defined(__HIPCC__)
// Forces a wave-uniform value (a kernel argument) into a scalar register here.
template <typename T>
__device__ __forceinline__ void PinScalar(const T &x) {
  asm volatile("" ::"s"(x));
}
#endif

// Everything a kernel reads about one dim lies together, and the dims a kernel usually has (one to three)
// come first: the scalar loads of the kernel arguments miss once per 64-byte line, one miss after the other
// when the index is not a compile-time constant, and that chain sits in front of a kernel's first load.
template <int NOPS>
struct NestArgs {
  struct Dim {
    FastDiv div;  // div.divisor is the extent
    int32_t strides[NOPS];
  };
  int32_t rank;
  Dim dims[kMaxRank];

#if defined(__HIPCC__)
  // Splits `index` over the dims (innermost last) and adds operand o's offset to off[o], o < N.
  template <int N>
  __device__ __forceinline__ void AddOffsets(uint32_t index, int32_t (&off)[N]) const {
    static_assert(N <= NOPS, "more offsets than operands");
    constexpr int kStatic = 4;  // dims handled with compile-time argument offsets
    // request the first three dims' descriptors in one batch (see the layout note above): left alone the
    // compiler fetches each field right before its use, one scalar-cache round trip after the other
    PinScalar(rank);
#pragma unroll
    for (int d = 0; d < 3; ++d) {
      PinScalar(dims[d].div.divisor);
      PinScalar(dims[d].div.multiplier);
      PinScalar(dims[d].div.shift);
#pragma unroll
      for (int o = 0; o < N; ++o) PinScalar(dims[d].strides[o]);
    }
    uint32_t rem = index;
    for (int d = rank - 1; d >= kStatic; --d) {
      uint32_t q, r;
      dims[d].div.DivMod(rem, q, r);
      rem = q;
#pragma unroll
      for (int o = 0; o < N; ++o) off[o] += static_cast<int32_t>(r) * dims[d].strides[o];
    }
#pragma unroll
    for (int d = kStatic - 1; d > 0; --d) {
      if (d < rank) {
        uint32_t q, r;
        dims[d].div.DivMod(rem, q, r);
        rem = q;
#pragma unroll
        for (int o = 0; o < N; ++o) off[o] += static_cast<int32_t>(r) * dims[d].strides[o];
      }
    }
#pragma unroll
    for (int o = 0; o < N; ++o) off[o] += static_cast<int32_t>(rem) * dims[0].strides[o];
  }
#endif
};

template <int NOPS>
inline NestArgs<NOPS> MakeNestArgs(const LoopNest &nest) {
  static_assert(NOPS <= kMaxOperands, "LoopNest holds strides for kMaxOperands operands");
  NestArgs<NOPS> a;
  std::memset(&a, 0, sizeof(a));
  a.rank = nest.rank;
  for (int i = 0; i < nest.rank; ++i) {
    a.dims[i].div = FastDiv(static_cast<uint32_t>(nest.shape[i]));
    for (int o = 0; o < NOPS; ++o) a.dims[i].strides[o] = static_cast<int32_t>(nest.strides[o][i]);
  }
  return a;
}

// ---- device-side reductions -------------------------------------------------

#if defined(__HIPCC__)
// The value of another lane through the data-parallel-primitive path of the vector ALU (a few cycles, against the
// round trip through the LDS crossbar that a shuffle by lane index costs).  `CTRL`: 0xB1 / 0x4E swap neighbours /
// pairs inside every four lanes, 0x141 / 0x140 mirror every 8 / 16 lanes.
template <int CTRL>
__device__ __forceinline__ float DppMove(float v) {
  const int bits = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(bits, bits, CTRL, 0xf, 0xf, false));
}

// Sum over every aligned group of W consecutive lanes (W a power of two), delivered to all lanes of the group.
// Every lane of the wave has to be active.
template <int W>
__device__ __forceinline__ float GroupSum(float v) {
  static_assert(W >= 1 && W <= kWave && (W & (W - 1)) == 0, "groups are powers of two");
  if constexpr (W >= 2) v += DppMove<0xB1>(v);
  if constexpr (W >= 4) v += DppMove<0x4E>(v);
  if constexpr (W >= 8) v += DppMove<0x141>(v);
  if constexpr (W >= 16) v += DppMove<0x140>(v);
  if constexpr (W >= 32) v += __shfl_xor(v, 16, kWave);
  if constexpr (W >= 64) v += __shfl_xor(v, 32, kWave);
  return v;
}

template <typename T, typename F>
__device__ __forceinline__ T WaveReduce(T v, F f) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    v = f(v, __shfl_xor(v, off, kWave));
  }
  return v;
}

struct SumOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct MaxOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

// Reduce across a block of NWAVES waves; `smem` needs NWAVES floats. All
// threads get the result.
template <int NWAVES, typename F>
__device__ __forceinline__ float BlockReduce(float v, F f, float *smem) {
  v = WaveReduce(v, f);
  if (NWAVES == 1) return v;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  __syncthreads();  // protect smem from a previous use
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float r = smem[0];
#pragma unroll
  for (int w = 1; w < NWAVES; ++w) r = f(r, smem[w]);
  return r;
}
#endif  // __HIPCC__

}  // namespace fl

#endif  // FLUIDML_AMD_CSRC_HIP_FL_COMMON_H_
