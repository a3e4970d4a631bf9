// 3x3 convolutions with unit stride and group 1 on the matrix cores, input staged once per workgroup.
// Reference: src/structure/kernel/kernel/conv.cpp:27-201 (ConvKernel::run, group == 1 branch :55-102; padded
// variant :230-280 -- the reference copies the input into a zero-filled scratch first, here padding reads as 0).
//
// The implicit-GEMM path of matmul.hip gathers the B operand element by element: every input value is fetched from
// global memory once per tap (nine times) by every workgroup that needs it, with an address decoded from k each time.
// Here a workgroup owns 64 filters x (4 x 16) or (8 x 16) output pixels of one image and walks the input channels eight at a time:
//   * the (4+2) x (16+2) input patch of the eight channels goes global -> registers -> LDS once (864 floats), next to
//     the 64 x 72 weights of those channels (contiguous runs of 72 floats per filter in the OIHW tensor);
//   * a wave owns 32 filters x 32 pixels (4 rows x 8 columns) and feeds v_mfma_f32_32x32x2_f32 straight from LDS: lane
//     (n = pixel, h = lane half) reads patch[channel 4h + c][py + kh][px + kw], lane (m = filter, h) reads
//     weights[m][(4h + c) * 9 + kh * 3 + kw] -- both addresses are a per-lane base plus a compile-time offset, so the
//     72 LDS reads of a chunk need no address arithmetic at all.  The order in which the 72 products of a chunk are
//     added is free, so the two lane halves simply take channels 0-3 and 4-7;
//   * LDS pitches (24 floats per patch row; 76 per weight row, read and written 128 bits at a time) keep the lanes of
//     an access in different banks;
//   * double-buffered LDS, the next two chunks' global loads are in flight while the current one is multiplied, one
//     barrier per chunk; two workgroups fit a compute unit and overlap each other's barriers;
//   * with few tiles (late layers at batch 1) the input channels of a tile are split over several workgroups, whose
//     partial tiles meet in the stream's workspace and are added in split order by the wave that arrives last;
//   * workgroup ids are dealt so that all filter tiles of a pixel tile run on one XCD, next to each other in time:
//     the patch is fetched into that L2 once.
// Bias and an elementwise chain (ReLU ...) are applied in registers before the stores, like in the other contractions.
//
// Opt-in bf16 (BF16 instantiations, FL_CONTRACT_BF16): the same workgroup tile and the same staging, 16 input channels per
// chunk, both operands rounded to bf16 (nearest even, hardware conversion) on their way into LDS and multiplied with
// v_mfma_f32_32x32x16_bf16, fp32 accumulation.  The 144 products of a chunk are split between the lane halves by channel
// (half h takes channels 8h .. 8h+7) and each half walks its 72 (channel, tap) pairs in the weights' own order: a lane's
// A operand of step s is 8 consecutive bf16 of its filter's row (one 128-bit LDS read), its B operand the 8 patch
// values at the matching (channel, kh, kw) offsets -- compile-time offsets from a per-lane base, eight 16-bit reads.
#include "fl_common.h"

namespace fl {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t Pack2(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, bf16x2{static_cast<__bf16>(lo), static_cast<__bf16>(hi)});
}
__device__ __forceinline__ uint16_t ToHalfWord(float f) { return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f)); }

constexpr int kTW = 16;                   // output columns per workgroup (rows: 4 per pixel tile of a wave, NV tiles)
constexpr int kFT = 64;                   // filters per workgroup
constexpr int kCC = 8;                    // input channels per chunk
constexpr int kPCols = kTW + 2;
constexpr int kPitch = 24;                // floats per patch row in LDS: rows 0..3 start in banks 0, 24, 16, 8
constexpr int kWPitch = 76;               // floats per filter in LDS (72 + 4: rows stay 16-byte aligned, 128-bit accesses
                                          // of consecutive filters fall into different bank groups)
constexpr int kWElems = kFT * kWPitch;    // 4864
constexpr int kThreads = 256;
constexpr int kSets = 2;                  // chunks on their way in registers (3: slower, 2905 against 2986 images/s on VGG-16 at batch 8)
constexpr int kWVecs = kFT * (kCC * 9 / 4);             // 1152 float4 of weights per chunk
constexpr int kWPer = (kWVecs + kThreads - 1) / kThreads;  // 5

struct HaloArgs {
  int32_t C, H, W, F, OH, OW;
  int32_t ph, pw;
  int32_t sXn, sXc, sXh, sXw;
  int32_t sWf;                 // floats between filters (weights are (c, kh, kw)-contiguous inside a filter)
  int32_t sOn, sOf, sOh, sOw;
  uint32_t tiles_h, tiles_w, tiles_f, tiles_pix;  // tiles_pix = images * tiles_h * tiles_w
  const float *bias;
  int32_t sB;
  // the input channels split over n_splits workgroups per tile (blockIdx.y), chunks_per_split chunks each; every wave
  // leaves its partial tiles in `partials` and the wave that arrives last at its counter adds them up in split order
  uint32_t n_splits;
  int32_t chunks_per_split;
  float *partials;
  uint32_t *counters;
  fl_ew_program chain;
};

// NV: pixel tiles (4 rows x 8 columns each) a wave owns, one below the other: the workgroup covers 4 NV x 16 pixels.
// With two, the weights a wave reads from LDS serve twice the products and a barrier separates twice the work.
// FEW: fewer than eight input channels (the first layer of an image network): one chunk whose missing channels read
// as zero; the filters' rows are then shorter than a chunk and not 16-byte aligned, so the weights are loaded
// value by value.
template <int NV, bool FEW>
__global__ __launch_bounds__(kThreads) void ConvHalo3x3Kernel(float *__restrict__ out, const float *__restrict__ in,
                                                              const float *__restrict__ weights, HaloArgs p) {
  constexpr int kTH = 4 * NV;
  constexpr int kPRows = kTH + 2;
  constexpr int kPlane = kPRows * kPitch;   // floats per channel of the patch: 144 (NV = 1), 240 (NV = 2)
  constexpr int kXElems = kCC * kPlane;
  constexpr int kStage = kXElems + kWElems; // 6016 / 6784 floats per buffer
  constexpr int kXItems = kCC * kPRows * kPCols;             // 864 / 1440 patch elements per chunk
  constexpr int kXPer = (kXItems + kThreads - 1) / kThreads; // 4 / 6
  __shared__ __attribute__((aligned(16))) float lds[2 * kStage];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int lrow = lane % 32, half = lane / 32;
  const int wm = wave / 2, wn = wave % 2;  // which 32 filters, which 8 pixel columns

  // ids are dealt round-robin to the 8 XCDs: give each XCD a contiguous run (all filter tiles of a pixel tile together)
  uint32_t bid = blockIdx.x;
  const uint32_t n_tiles = p.tiles_pix * p.tiles_f;
  if (n_tiles % 8 == 0) bid = (bid % 8) * (n_tiles / 8) + bid / 8;
  const uint32_t f_tile = bid % p.tiles_f;
  uint32_t pix = bid / p.tiles_f;
  const uint32_t tw = pix % p.tiles_w;
  pix /= p.tiles_w;
  const uint32_t th = pix % p.tiles_h;
  const uint32_t img = pix / p.tiles_h;
  const int f0 = static_cast<int>(f_tile) * kFT, oh0 = static_cast<int>(th) * kTH, ow0 = static_cast<int>(tw) * kTW;

  // what this thread moves per chunk: kWPer float4 of weights and kXPer patch elements
  const float *w_src[kWPer];
  int w_dst[kWPer];
  bool w_ok[kWPer];
#pragma unroll
  for (int t = 0; t < kWPer; ++t) {
    const int i = tid + t * kThreads;
    const int f = i / 18, q = i % 18;
    w_ok[t] = i < kWVecs && f0 + f < p.F;
    w_src[t] = weights + static_cast<int64_t>(min(f0 + f, p.F - 1)) * p.sWf + q * 4;
    w_dst[t] = f * kWPitch + q * 4;
  }
  const float *x_src[kXPer];
  int x_dst[kXPer];
  bool x_ok[kXPer];
  const float *image = in + static_cast<int64_t>(img) * p.sXn;
#pragma unroll
  for (int t = 0; t < kXPer; ++t) {
    const int i = tid + t * kThreads;
    const int ch = i / (kPRows * kPCols), rem = i % (kPRows * kPCols);
    const int r = rem / kPCols, s = rem % kPCols;
    const int ih = oh0 - p.ph + r, iw = ow0 - p.pw + s;
    x_ok[t] = i < kXItems && static_cast<uint32_t>(ih) < static_cast<uint32_t>(p.H) &&
              static_cast<uint32_t>(iw) < static_cast<uint32_t>(p.W) && (!FEW || ch < p.C);
    x_src[t] = image + (x_ok[t] ? static_cast<int64_t>(ch) * p.sXc + ih * p.sXh + iw * p.sXw : 0);
    x_dst[t] = i < kXItems ? ch * kPlane + r * kPitch + s : -1;
  }

  // kSets chunks are on their way in registers (chunk i of this workgroup in set i % kSets) while another is
  // multiplied from LDS: a chunk's loads have kSets multiplication phases to arrive, not one
  constexpr int kS = FEW ? 1 : kSets;  // (a single chunk there)
  floatx4 wr[kS][kWPer];
  float xr[kS][kXPer];
  auto load_chunk = [&](int c, auto set_c) {
    constexpr int S = decltype(set_c)::value;
    const int c0 = c * kCC;
#pragma unroll
    for (int t = 0; t < kWPer; ++t) {
      if constexpr (FEW) {
        const int q4 = ((tid + t * kThreads) % 18) * 4, n_w = p.C * 9;  // position of the piece inside the filter's row
        wr[S][t] = floatx4{w_ok[t] && q4 < n_w ? w_src[t][0] : 0.0f, w_ok[t] && q4 + 1 < n_w ? w_src[t][1] : 0.0f,
                           w_ok[t] && q4 + 2 < n_w ? w_src[t][2] : 0.0f, w_ok[t] && q4 + 3 < n_w ? w_src[t][3] : 0.0f};
      } else {
        wr[S][t] = w_ok[t] ? *reinterpret_cast<const floatx4 *>(w_src[t] + c0 * 9) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
#pragma unroll
    for (int t = 0; t < kXPer; ++t) xr[S][t] = x_ok[t] ? x_src[t][static_cast<int64_t>(c0) * p.sXc] : 0.0f;
  };
  auto store_chunk = [&](auto set_c, auto buf_c) {
    constexpr int S = decltype(set_c)::value;
    float *xs = lds + decltype(buf_c)::value * kStage;
    float *ws = xs + kXElems;
#pragma unroll
    for (int t = 0; t < kWPer; ++t) {
      if (tid + t * kThreads < kWVecs) *reinterpret_cast<floatx4 *>(ws + w_dst[t]) = wr[S][t];
    }
#pragma unroll
    for (int t = 0; t < kXPer; ++t) {
      if (x_dst[t] >= 0) xs[x_dst[t]] = xr[S][t];
    }
  };

  floatx16 acc[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[v][e] = 0.0f;
  const int py = lrow / 8, px = lrow % 8 + 8 * wn;
  const int a_base = (wm * 32 + lrow) * kWPitch + half * 36;
  const int b_base = half * 4 * kPlane + py * kPitch + px;

  const int all_chunks = FEW ? 1 : p.C / kCC;
  const int c_first = !FEW && p.n_splits > 1 ? static_cast<int>(blockIdx.y) * p.chunks_per_split : 0;
  const int n_chunks = !FEW && p.n_splits > 1 ? min(all_chunks, c_first + p.chunks_per_split) : all_chunks;
  // chunk c (the i-th of this workgroup), held in LDS buffer i % 2 and come through register set i % kSets: request
  // chunk c + kSets into those registers, multiply, move chunk c + 1 (requested kSets - 1 phases ago) from its
  // registers to the other buffer
  auto phase = [&](int c, auto idx_c) {
    constexpr int I = decltype(idx_c)::value;
    using Regs = std::integral_constant<int, I % kS>;
    using NextRegs = std::integral_constant<int, (I + 1) % kS>;
    using NextBuf = std::integral_constant<int, (I + 1) % 2>;
    if (c + kS < n_chunks) load_chunk(c + kS, Regs{});
    const float *xs = lds + (I % 2) * kStage;
    const float *ws = xs + kXElems;
#pragma unroll
    for (int g = 0; g < 9; ++g) {
      const floatx4 a4 = *reinterpret_cast<const floatx4 *>(ws + a_base + 4 * g);
      const float a[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int j = 4 * g + e, c4 = j / 9, kh = (j % 9) / 3, kw = j % 3;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
          const float b = xs[b_base + c4 * kPlane + (kh + 4 * v) * kPitch + kw];
          acc[v] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b, acc[v], 0, 0, 0);
        }
      }
    }
    if (c + 1 < n_chunks) store_chunk(NextRegs{}, NextBuf{});
    // one barrier per chunk: the buffer written here was last read in the previous phase, and every wave
    // passed the previous barrier only after finishing that read
    __syncthreads();
  };
  StaticFor<kS>([&](auto k) {
    if (c_first + decltype(k)::value < n_chunks) load_chunk(c_first + decltype(k)::value, k);
  });
  store_chunk(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
  __syncthreads();
  constexpr int kPeriod = kS % 2 == 0 ? kS : 2 * kS;  // after this many phases registers and buffer repeat
  for (int c = c_first; c < n_chunks; c += kPeriod) {
    StaticFor<kPeriod>([&](auto k) {
      if (c + decltype(k)::value < n_chunks) phase(c + decltype(k)::value, k);
    });
  }

  // ---- channels split over workgroups: combine the partial tiles ----------------------------------------------
  // Each wave runs the hand-off on its own slots and its own counter, so no workgroup barrier is involved.  The
  // partial tiles travel through device-coherent accesses (agent-scope atomics: write-through stores, loads that
  // miss in the per-XCD L2).  Release: the wave waits until every vector memory operation it has issued is
  // acknowledged (s_waitcnt vmcnt(0); stores count in vmcnt on gfx9) before it counts its arrival; the "memory"
  // clobber keeps the compiler from moving the stores below the wait or the counter update above it.  Acquire: the
  // loads of the partial tiles follow the branch on the counter's returned value, which the wave has to wait for.
  // The sums run in split order, so the result does not depend on which workgroup arrives last.
  if (!FEW && p.n_splits > 1) {  // (a single chunk is never split)
    const uint32_t n_splits = p.n_splits;
    const uint32_t wslot = blockIdx.x * 4 + wave;
    float *mine = p.partials + (static_cast<size_t>(wslot) * n_splits + blockIdx.y) * (NV * 1024);
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        __hip_atomic_store(mine + v * 1024 + e * 64 + lane, acc[v][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    uint32_t arrived = 0;
    if (lane == 0) arrived = __hip_atomic_fetch_add(&p.counters[wslot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    arrived = __shfl(arrived, 0);
    if (arrived != n_splits - 1) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // compiler ordering only: no instruction on gfx9
    if (lane == 0) __hip_atomic_store(&p.counters[wslot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float *all = p.partials + static_cast<size_t>(wslot) * n_splits * (NV * 1024);
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[v][e] = 0.0f;
    // the loads of several splits are in flight together (one round trip for all of them); the sums still run in
    // split order
    constexpr uint32_t kAhead = 8 / NV;
    for (uint32_t z0 = 0; z0 < n_splits; z0 += kAhead) {
      float part[kAhead][NV][16];
#pragma unroll
      for (uint32_t u = 0; u < kAhead; ++u) {
        const uint32_t z = z0 + u < n_splits ? z0 + u : z0;  // repeats a valid slot, ignored below
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            part[u][v][e] = __hip_atomic_load(all + static_cast<size_t>(z) * (NV * 1024) + v * 1024 + e * 64 + lane,
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
      }
#pragma unroll
      for (uint32_t u = 0; u < kAhead; ++u) {
        if (z0 + u < n_splits) {
#pragma unroll
          for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[v][e] += part[u][v][e];
        }
      }
    }
  }

  // ---- epilogue: bias, elementwise chain, stores -------------------------------------------------------------
  float bias_v[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int f = f0 + wm * 32 + (e / 4) * 8 + half * 4 + (e % 4);
    bias_v[e] = p.bias != nullptr && f < p.F ? p.bias[f * p.sB] : 0.0f;
  }
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int oh = oh0 + py + 4 * v, ow = ow0 + px;
    float vals[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) vals[e] = acc[v][e] + bias_v[e];
    if (p.chain.n != 0) RunChainBlock<16>(p.chain, vals);
    if (oh < p.OH && ow < p.OW) {
      float *dst = out + static_cast<int64_t>(img) * p.sOn + static_cast<int64_t>(oh) * p.sOh + static_cast<int64_t>(ow) * p.sOw;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int f = f0 + wm * 32 + (e / 4) * 8 + half * 4 + (e % 4);
        if (f < p.F) dst[static_cast<int64_t>(f) * p.sOf] = vals[e];
      }
    }
  }
}

// ---- bf16 operands -----------------------------------------------------------------------------------------------
constexpr int kCC16 = 16;                        // input channels per chunk
constexpr int kWPitch16 = 152;                   // 16-bit words per filter in LDS: 144 + 8 (76 32-bit words, as above)
constexpr int kWElems16 = kFT * kWPitch16;
constexpr int kWVecs16 = kFT * (kCC16 * 9 / 4);  // 2304 float4 of weights per chunk
constexpr int kWPer16 = kWVecs16 / kThreads;     // 9

template <int NV>
__global__ __launch_bounds__(kThreads) void ConvHalo3x3Bf16Kernel(float *__restrict__ out, const float *__restrict__ in,
                                                                  const float *__restrict__ weights, HaloArgs p) {
  constexpr int kTH = 4 * NV;
  constexpr int kPRows = kTH + 2;
  constexpr int kPlane = kPRows * kPitch + 8;   // 16-bit words per channel: the two lane halves (8 channels apart) land
                                                // in different halves of the banks
  constexpr int kXElems = kCC16 * kPlane;
  constexpr int kStage = kXElems + kWElems16;   // 16-bit words per buffer (12,160 / 13,696)
  constexpr int kXItems = kCC16 * kPRows * kPCols;
  constexpr int kXPer = (kXItems + kThreads - 1) / kThreads;  // 7 / 12
  __shared__ __attribute__((aligned(16))) uint16_t lds[2 * kStage];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int lrow = lane % 32, half = lane / 32;
  const int wm = wave / 2, wn = wave % 2;

  uint32_t bid = blockIdx.x;
  const uint32_t n_tiles = p.tiles_pix * p.tiles_f;
  if (n_tiles % 8 == 0) bid = (bid % 8) * (n_tiles / 8) + bid / 8;
  const uint32_t f_tile = bid % p.tiles_f;
  uint32_t pix = bid / p.tiles_f;
  const uint32_t tw = pix % p.tiles_w;
  pix /= p.tiles_w;
  const uint32_t th = pix % p.tiles_h;
  const uint32_t img = pix / p.tiles_h;
  const int f0 = static_cast<int>(f_tile) * kFT, oh0 = static_cast<int>(th) * kTH, ow0 = static_cast<int>(tw) * kTW;

  const float *w_src[kWPer16];
  int w_dst[kWPer16];
  bool w_ok[kWPer16];
#pragma unroll
  for (int t = 0; t < kWPer16; ++t) {
    const int i = tid + t * kThreads;
    const int f = i / 36, q = i % 36;
    w_ok[t] = f0 + f < p.F;
    w_src[t] = weights + static_cast<int64_t>(min(f0 + f, p.F - 1)) * p.sWf + q * 4;
    w_dst[t] = f * kWPitch16 + q * 4;
  }
  const float *x_src[kXPer];
  int x_dst[kXPer];
  bool x_ok[kXPer];
  const float *image = in + static_cast<int64_t>(img) * p.sXn;
#pragma unroll
  for (int t = 0; t < kXPer; ++t) {
    const int i = tid + t * kThreads;
    const int ch = i / (kPRows * kPCols), rem = i % (kPRows * kPCols);
    const int r = rem / kPCols, s = rem % kPCols;
    const int ih = oh0 - p.ph + r, iw = ow0 - p.pw + s;
    x_ok[t] = i < kXItems && static_cast<uint32_t>(ih) < static_cast<uint32_t>(p.H) &&
              static_cast<uint32_t>(iw) < static_cast<uint32_t>(p.W);
    x_src[t] = image + (x_ok[t] ? static_cast<int64_t>(ch) * p.sXc + ih * p.sXh + iw * p.sXw : 0);
    x_dst[t] = i < kXItems ? ch * kPlane + r * kPitch + s : -1;
  }

  floatx4 wr[kSets][kWPer16];
  float xr[kSets][kXPer];
  auto load_chunk = [&](int c, auto set_c) {
    constexpr int S = decltype(set_c)::value;
    const int c0 = c * kCC16;
#pragma unroll
    for (int t = 0; t < kWPer16; ++t) {
      wr[S][t] = w_ok[t] ? *reinterpret_cast<const floatx4 *>(w_src[t] + c0 * 9) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int t = 0; t < kXPer; ++t) xr[S][t] = x_ok[t] ? x_src[t][static_cast<int64_t>(c0) * p.sXc] : 0.0f;
  };
  auto store_chunk = [&](auto set_c, auto buf_c) {
    constexpr int S = decltype(set_c)::value;
    uint16_t *xs = lds + decltype(buf_c)::value * kStage;
    uint16_t *ws = xs + kXElems;
#pragma unroll
    for (int t = 0; t < kWPer16; ++t) {
      *reinterpret_cast<u32x2 *>(ws + w_dst[t]) = u32x2{Pack2(wr[S][t].x, wr[S][t].y), Pack2(wr[S][t].z, wr[S][t].w)};
    }
#pragma unroll
    for (int t = 0; t < kXPer; ++t) {
      if (x_dst[t] >= 0) xs[x_dst[t]] = ToHalfWord(xr[S][t]);
    }
  };

  floatx16 acc[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[v][e] = 0.0f;
  const int py = lrow / 8, px = lrow % 8 + 8 * wn;
  const int a_base = (wm * 32 + lrow) * kWPitch16 + half * 72;
  const int b_base = half * 8 * kPlane + py * kPitch + px;

  const int all_chunks = p.C / kCC16;
  const int c_first = p.n_splits > 1 ? static_cast<int>(blockIdx.y) * p.chunks_per_split : 0;
  const int n_chunks = p.n_splits > 1 ? min(all_chunks, c_first + p.chunks_per_split) : all_chunks;
  auto phase = [&](int c, auto idx_c) {
    constexpr int I = decltype(idx_c)::value;
    using Regs = std::integral_constant<int, I % kSets>;
    using NextRegs = std::integral_constant<int, (I + 1) % kSets>;
    using NextBuf = std::integral_constant<int, (I + 1) % 2>;
    if (c + kSets < n_chunks) load_chunk(c + kSets, Regs{});
    const uint16_t *xs = lds + (I % 2) * kStage;
    const uint16_t *ws = xs + kXElems;
#pragma unroll
    for (int g = 0; g < 9; ++g) {
      const u32x4 a8 = *reinterpret_cast<const u32x4 *>(ws + a_base + 8 * g);
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        uint32_t h[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int j = 8 * g + e, c8 = j / 9, kh = (j % 9) / 3, kw = j % 3;
          h[e] = xs[b_base + c8 * kPlane + (kh + 4 * v) * kPitch + kw];
        }
        const u32x4 b8 = {h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16};
        acc[v] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a8), __builtin_bit_cast(bf16x8, b8), acc[v], 0, 0, 0);
      }
    }
    if (c + 1 < n_chunks) store_chunk(NextRegs{}, NextBuf{});
    __syncthreads();
  };
  StaticFor<kSets>([&](auto k) {
    if (c_first + decltype(k)::value < n_chunks) load_chunk(c_first + decltype(k)::value, k);
  });
  store_chunk(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
  __syncthreads();
  for (int c = c_first; c < n_chunks; c += kSets) {
    StaticFor<kSets>([&](auto k) {
      if (c + decltype(k)::value < n_chunks) phase(c + decltype(k)::value, k);
    });
  }

  // ---- channels split over workgroups: the hand-off of the fp32 kernel above -------------------------------------
  if (p.n_splits > 1) {
    const uint32_t n_splits = p.n_splits;
    const uint32_t wslot = blockIdx.x * 4 + wave;
    float *mine = p.partials + (static_cast<size_t>(wslot) * n_splits + blockIdx.y) * (NV * 1024);
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        __hip_atomic_store(mine + v * 1024 + e * 64 + lane, acc[v][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    uint32_t arrived = 0;
    if (lane == 0) arrived = __hip_atomic_fetch_add(&p.counters[wslot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    arrived = __shfl(arrived, 0);
    if (arrived != n_splits - 1) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // compiler ordering only
    if (lane == 0) __hip_atomic_store(&p.counters[wslot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float *all = p.partials + static_cast<size_t>(wslot) * n_splits * (NV * 1024);
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[v][e] = 0.0f;
    for (uint32_t z = 0; z < n_splits; ++z) {  // in split order
#pragma unroll
      for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          acc[v][e] += __hip_atomic_load(all + static_cast<size_t>(z) * (NV * 1024) + v * 1024 + e * 64 + lane, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
        }
    }
  }

  float bias_v[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int f = f0 + wm * 32 + (e / 4) * 8 + half * 4 + (e % 4);
    bias_v[e] = p.bias != nullptr && f < p.F ? p.bias[f * p.sB] : 0.0f;
  }
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int oh = oh0 + py + 4 * v, ow = ow0 + px;
    float vals[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) vals[e] = acc[v][e] + bias_v[e];
    if (p.chain.n != 0) RunChainBlock<16>(p.chain, vals);
    if (oh < p.OH && ow < p.OW) {
      float *dst = out + static_cast<int64_t>(img) * p.sOn + static_cast<int64_t>(oh) * p.sOh + static_cast<int64_t>(ow) * p.sOw;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int f = f0 + wm * 32 + (e / 4) * 8 + half * 4 + (e % 4);
        if (f < p.F) dst[static_cast<int64_t>(f) * p.sOf] = vals[e];
      }
    }
  }
}

// Environment FLUIDML_CONV_HALO=0 keeps every convolution on the implicit-GEMM path.
bool HaloEnabled() {
  const char *v = std::getenv("FLUIDML_CONV_HALO");  // (read at every call)
  return v == nullptr || std::strtol(v, nullptr, 10) != 0;
}

}  // namespace

// FL_ERR_UNSUPPORTED (nothing launched) when the convolution does not fit this kernel: the caller goes on to the
// implicit-GEMM path.  Operands were validated by the caller.
int ConvHalo3x3(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out,
                const int64_t *pads, const int64_t *strides, const int64_t *dilations, const fl_ew_program *chain,
                void *stream, bool bf16) {
  if (!HaloEnabled() || out->rank != 4) return FL_ERR_UNSUPPORTED;
  if (weights->shape[2] != 3 || weights->shape[3] != 3) return FL_ERR_UNSUPPORTED;
  for (int d = 0; d < 2; ++d) {
    if ((strides && strides[d] != 1) || (dilations && dilations[d] != 1)) return FL_ERR_UNSUPPORTED;
  }
  const int64_t N = in->shape[0], C = in->shape[1], H = in->shape[2], W = in->shape[3];
  const int64_t F = out->shape[1], OH = out->shape[2], OW = out->shape[3];
  const bool few = C < kCC;
  if ((C % kCC != 0 && !few) || F < 32) return FL_ERR_UNSUPPORTED;
  // bf16 operands: chunks of 16 channels (other channel counts, and the first layer's few channels, stay fp32)
  const bool half_words = bf16 && !few && C % kCC16 == 0;
  const int64_t chunk = half_words ? kCC16 : kCC;
  // weights (c, kh, kw)-contiguous inside a filter, filters 16-byte aligned
  if (weights->strides[3] != 1 || weights->strides[2] != 3 || weights->strides[1] != 9) return FL_ERR_UNSUPPORTED;
  if (!few && (weights->strides[0] % 4 != 0 || !IsAligned(weights->base, 16))) return FL_ERR_UNSUPPORTED;
  if (Numel(in) > 0x7fffffff || Numel(out) > 0x7fffffff || Numel(weights) > 0x7fffffff) return FL_ERR_UNSUPPORTED;
  const int64_t ph = pads ? pads[0] : 0, pw = pads ? pads[1] : 0;
  if (ph < 0 || pw < 0 || ph > 2 || pw > 2) return FL_ERR_UNSUPPORTED;
  HaloArgs p;
  std::memset(&p, 0, sizeof(p));
  p.C = static_cast<int32_t>(C), p.H = static_cast<int32_t>(H), p.W = static_cast<int32_t>(W);
  p.F = static_cast<int32_t>(F), p.OH = static_cast<int32_t>(OH), p.OW = static_cast<int32_t>(OW);
  p.ph = static_cast<int32_t>(ph), p.pw = static_cast<int32_t>(pw);
  p.sXn = static_cast<int32_t>(in->strides[0]), p.sXc = static_cast<int32_t>(in->strides[1]);
  p.sXh = static_cast<int32_t>(in->strides[2]), p.sXw = static_cast<int32_t>(in->strides[3]);
  p.sWf = static_cast<int32_t>(weights->strides[0]);
  p.sOn = static_cast<int32_t>(out->strides[0]), p.sOf = static_cast<int32_t>(out->strides[1]);
  p.sOh = static_cast<int32_t>(out->strides[2]), p.sOw = static_cast<int32_t>(out->strides[3]);
  // two pixel tiles per wave when the rows divide evenly and plenty of workgroups remain (measured at batch 8:
  // 64 x 224 x 224 with 3136 such workgroups 89 -> 96 TFLOP/s, 128 x 112 x 112 with 1568 98 -> 99, but
  // 256 x 56 x 56 with 896 98 -> 94)
  const int64_t tiles_f64 = (F + kFT - 1) / kFT, tiles_w64 = (OW + kTW - 1) / kTW;
  const int nv = (OH % 8 == 0 && N * (OH / 8) * tiles_w64 * tiles_f64 >= 1500) ? 2 : 1;
  const int64_t kTH = 4 * nv;
  p.tiles_h = static_cast<uint32_t>((OH + kTH - 1) / kTH);
  p.tiles_w = static_cast<uint32_t>((OW + kTW - 1) / kTW);
  p.tiles_f = static_cast<uint32_t>((F + kFT - 1) / kFT);
  const int64_t tiles_pix = N * p.tiles_h * p.tiles_w;
  const int64_t n_tiles = tiles_pix * p.tiles_f;
  // worth it when the pixel tiles are mostly full and there are enough workgroups to fill the chip
  // (14 x 14 images fill 77 % of their tiles: without a split measured slower than the implicit-GEMM path, 113.7
  // against 107.9 us)
  const double fill = static_cast<double>(OH * OW) / static_cast<double>(p.tiles_h * kTH * p.tiles_w * kTW);
  // (workgroups: 224 at batch 1 on 256 x 56 x 56 still win, 40.7 -> 30.3 us with 128 input channels and 56.7 -> 54.3
  // with 256; 112 unsplit on 512 x 28 x 28 lose against the implicit GEMM with K split over workgroups, 60 -> 100 us)
  // Few tiles and many channels (late layers at batch 1): the chunks of a tile go to several workgroups, aiming at
  // two workgroups per compute unit (a workgroup is one wave per SIMD: a second one fills its barriers and loads).
  // Measured on VGG-16 at batch 1 (1474 -> 1671 images/s; with the second chunk in flight 1726): 512 x 14 x 14 with
  // 32 tiles 34 -> 23 us, 512 x 28 x 28 with 112 tiles 61 -> 51 us, 256 x 56 x 56 with 224 tiles 54 -> 50 us; aiming
  // at 256, 384, 640 or 1024 workgroups, or fewer than 4 chunks per workgroup, is slower; with one or two pixel tiles
  // per wave and 1, 2, 3, 4 or 6 splits forced on every layer, only 64 x 224 x 224 gains on this rule (two tiles: 50 ->
  // 46 us).
  constexpr int64_t kTargetWorkgroups = 512, kMinChunks = 8;
  int64_t splits = 1;
  const int64_t all_chunks = few ? 1 : C / chunk;
  if (n_tiles > 0 && n_tiles < kTargetWorkgroups && n_tiles * 4 <= static_cast<int64_t>(kWorkspaceTiles)) {
    // (one counter per wave of a tile, one workspace slot per wave, pixel tile and split)
    splits = std::min<int64_t>({kTargetWorkgroups / n_tiles, all_chunks / kMinChunks,
                                static_cast<int64_t>(kWorkspaceTiles) / (n_tiles * 4 * nv)});
  }
  StreamWorkspace *ws = splits >= 2 ? GetStreamWorkspace(AsStream(stream)) : nullptr;
  if (ws == nullptr) splits = 1;
  // (split, 14 x 14 images with 77 % of their tiles filled win against the implicit GEMM as well: 34 -> 23 us)
  if (n_tiles > 0x7fffffff || n_tiles * splits < 192 || fill < (splits > 1 ? 0.75 : 0.8)) return FL_ERR_UNSUPPORTED;
  if (splits > 1) {
    p.chunks_per_split = static_cast<int32_t>((all_chunks + splits - 1) / splits);
    p.n_splits = static_cast<uint32_t>((all_chunks + p.chunks_per_split - 1) / p.chunks_per_split);
    p.partials = ws->partials;
    p.counters = ws->counters;
  } else {
    p.n_splits = 1;
  }
  p.tiles_pix = static_cast<uint32_t>(tiles_pix);
  if (bias != nullptr) {
    p.bias = static_cast<const float *>(bias->base);
    p.sB = static_cast<int32_t>(bias->strides[0]);
  }
  if (chain != nullptr) p.chain = *chain;
#define FL_HALO(NV_, FEW_)                                                                                          \
  FL_LAUNCH((ConvHalo3x3Kernel<NV_, FEW_>), dim3(static_cast<uint32_t>(n_tiles), p.n_splits), dim3(kThreads), 0, AsStream(stream), \
            static_cast<float *>(out->base), static_cast<const float *>(in->base),                                  \
            static_cast<const float *>(weights->base), p)
  if (half_words) {
    if (nv == 2) {
      FL_LAUNCH((ConvHalo3x3Bf16Kernel<2>), dim3(static_cast<uint32_t>(n_tiles), p.n_splits), dim3(kThreads), 0, AsStream(stream),
                static_cast<float *>(out->base), static_cast<const float *>(in->base), static_cast<const float *>(weights->base), p);
    } else {
      FL_LAUNCH((ConvHalo3x3Bf16Kernel<1>), dim3(static_cast<uint32_t>(n_tiles), p.n_splits), dim3(kThreads), 0, AsStream(stream),
                static_cast<float *>(out->base), static_cast<const float *>(in->base), static_cast<const float *>(weights->base), p);
    }
  } else if (few) {
    if (nv == 2) FL_HALO(2, true);
    else FL_HALO(1, true);
  } else if (nv == 2) {
    FL_HALO(2, false);
  } else {
    FL_HALO(1, false);
  }
#undef FL_HALO
  return LaunchStatus();
}

}  // namespace fl
