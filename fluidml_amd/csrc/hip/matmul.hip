// fp32 contractions on the CDNA4 matrix cores: MatMul (NumPy batch broadcast)
// and Gemm (rank-2 with alpha/beta/bias epilogue).
// Reference: src/structure/kernel/kernel/matmul.cpp:28-59, gemm.cpp:39-182,
// utils.cpp:64-147 (broadcast maps).
//
// C[b..., m, n] = sum_k A[b..., m, k] * B[b..., k, n] over arbitrary element
// strides: the layout the planner picked only decides which of (m,k) resp.
// (k,n) is walked by the 128-bit global loads and how the tile sits in LDS.
//
//   * v_mfma_f32_32x32x2_f32 (64 lanes x 1 A value, 1 B value -> 32x32 fp32
//     accumulators, 16 per lane); a wave owns TM x TN such tiles;
//   * tiles are staged global -> registers -> LDS with double buffering, one
//     barrier per K chunk; an operand that is k-contiguous in memory is kept
//     [x][k] (+4 pad, 128-bit LDS reads), otherwise [k][x] (32-bit reads);
//   * each lane half handles 4 consecutive k per group of 8 (the k order inside
//     a sum is free), so the [x][k] layout needs one ds_read_b128 per 4 MFMAs;
//   * small problems split each K chunk over the waves of a workgroup and
//     combine the partial tiles through LDS, so M=128-row problems still put
//     4 waves on every tile;
//   * workgroup ids are folded so that consecutive tiles land on one XCD and
//     share its L2.
//
// A second, opt-in path (BF16 instantiations) rounds both operands to bf16 (round to nearest even) once, on their
// way from registers into LDS, keeps the staged tiles as bf16 (half the LDS traffic) and multiplies them with
// v_mfma_f32_32x32x16_bf16; accumulation stays fp32.  A lane feeds the instruction 8 consecutive k of its row of A and
// of its column of B (lane half h holds k = 8h..8h+7 of a group of 16): one 128-bit LDS read where the tile is kept
// k-contiguous ([m][k], [n][k]), eight 16-bit reads where it is kept the other way ([k][m], [k][n]: the operand's
// fast dimension in memory is not k, and transposing 2-byte elements on the way into LDS would cost 8-way bank
// conflicts).  One bf16 instruction replaces eight fp32 ones at half their duration.
#include <algorithm>
#include <cstddef>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>

#include "fl_common.h"

namespace fl {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef short bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// float -> bf16 bits, round to nearest even (NaN stays NaN): the hardware conversion (v_cvt_pk_bf16_f32, two values
// per instruction)
__device__ __forceinline__ short ToBf16(float f) { return __builtin_bit_cast(short, static_cast<__bf16>(f)); }
__device__ __forceinline__ uint32_t PackBf16(float lo, float hi) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, bf16x2{static_cast<__bf16>(lo), static_cast<__bf16>(hi)});
}

// Geometry of a convolution run as an implicit GEMM: M = output channels, N = images x output pixels,
// K = input channels x kernel taps.  B[k][n] is gathered from the input on the fly (padding reads as 0),
// C[m][n] is scattered to out[image, m, oh, ow].  1-d convolutions use H = OH = KH = 1.
struct ConvGeom {
  int32_t H, W;                  // input extents
  int32_t sh, sw, dh, dw, ph, pw;
  int32_t sXn, sXc, sXh, sXw;    // input element strides
  int32_t sOn, sOh, sOw;         // output element strides (the channel stride is sCm)
  FastDiv div_ohw, div_ow;       // n -> (image, oh, ow)
  FastDiv div_khw, div_kw;       // k -> (channel, kh, kw)
};

// Batch dims of a contraction after merging (operand 0 = C, 1 = A, 2 = B), innermost last.  Kept small and
// statically indexed: the kernel's scalar loads of its arguments are a serial chain of cache misses otherwise.
constexpr int kMaxBatchDims = 4;
struct BatchArgs {
  int32_t rank;  // 0: a single batch element
  FastDiv div[kMaxBatchDims];
  int32_t strides[3][kMaxBatchDims];
};

// Kernel arguments.  Every workgroup needs the first block before it can issue its first load, and a cold
// 64-byte line of kernel arguments costs a few hundred nanoseconds: what every launch reads comes first and
// is packed (two lines), what the EXTRA instantiations read follows (the next line and a half), and what only some
// launches read (batch dims, chain, siblings, convolution geometry) comes last.
struct MatmulArgs {
  int32_t M, N, K;
  int32_t sAm, sAk, sBk, sBn, sCm, sCn;
  uint32_t tiles_m, tiles_n;
  // split K over `n_splits` workgroups per tile (blockIdx.z): each takes `chunks_per_split` chunks, writes its
  // partial tile to `partials`, and the workgroup that arrives last at `counters[tile]` adds them up in split order
  uint32_t n_splits;
  int32_t chunks_per_split;
  // sibling contractions that share A and every extent, one per blockIdx.y (n_groups <= 1: none; batch
  // dims are then absent).  Member 0 uses the fields here, member g > 0 the entries g - 1 of the g* arrays.
  int32_t n_groups;
  // optional two-level column addressing of C: column n lives at (n / n_inner) * sCn_outer + (n % n_inner) * sCn
  // (the last output dim reshaped into two dims that a transpose moved apart); n_inner == 0: n * sCn
  int32_t n_inner, sCn_outer;
  // epilogue: C = ca * acc + cb * bias[m * sDm + n * sDn]   (bias may be null)
  const float *bias;
  int32_t sDm, sDn;
  float ca, cb;
  float *partials;
  uint32_t *counters;
  // copies of batch.rank and chain.n (set at launch), so that a launch without batch dims or chain never touches
  // the lines those live in
  int32_t batch_rank, chain_n;
  // EXTRA == 1 instantiations only, one batch element: a LayerNormalization kept out of memory (fl_norm_fusion).
  // ln_mode 1: A holds the un-normalised tensor, the epilogue turns acc into rstd * (acc - mean * c1[n]) + bias[n];
  // ln_mode 2: the addend does, and enters as (t - mean) * rstd * scale[n] + shift[n].  Row statistics come as
  // ln_parts (mean, M2) pairs per row, each over 32 consecutive columns of the ln_width wide tensor.
  int32_t ln_mode, ln_parts, ln_width;
  float ln_eps;
  // ---- byte 128 ----
  // EXTRA instantiations only (plain contraction, B kept [k][n]), all optional:
  // a tensor with the strides of C, added to the value after the chain (read at the element offset the value is
  // stored at);
  const float *addend;
  // a second one, added after the first;
  const float *addend2;
  // one batch element: row k of B is multiplied by k_scale[k * sKs] while it is staged, each product rounded like
  // a separate Mul kernel's
  const float *k_scale;
  int32_t sKs;
  float ln_inv_width;  // (1 / ln_width, rounded once on the host)
  const float *ln_stats;
  const float *ln_c1;                 // mode 1, member 0 (members g > 0: g_ln_c1[g - 1])
  const float *ln_scale, *ln_shift;   // mode 2
  // ---- byte 192 ----
  float *ln_stats_out;                // non-null: (mean, M2) of every 32-column run of C's rows, ceil(N / 32) per row
  int32_t ln_s_scale, ln_s_shift, ln_s_c1;  // element strides of the three vectors
  int32_t addend_is_factor;                 // EXTRA: the value is multiplied by `addend` instead
  FastDiv div_inner;
  const float *g_ln_c1[3];
  const float *gB[3];
  float *gC[3];
  const float *gbias[3];
  int32_t g_sCm[3], g_sCn[3], g_sCn_outer[3];
  BatchArgs batch;
  // optional elementwise chain applied after the bias (chain.n == 0: none)
  fl_ew_program chain;
  ConvGeom conv;  // read by the CONV instantiations only
};
static_assert(offsetof(MatmulArgs, addend) == 128 && offsetof(MatmulArgs, ln_stats_out) == 192,
              "the packing of the kernel arguments into lines is deliberate");

inline int MakeBatchArgs(const LoopNest &nest, int64_t n_batch, BatchArgs *b) {
  std::memset(b, 0, sizeof(*b));
  if (n_batch == 1) return FL_OK;
  if (nest.rank > kMaxBatchDims) return FL_ERR_UNSUPPORTED;
  b->rank = nest.rank;
  for (int i = 0; i < nest.rank; ++i) {
    b->div[i] = FastDiv(static_cast<uint32_t>(nest.shape[i]));
    for (int o = 0; o < 3; ++o) b->strides[o][i] = static_cast<int32_t>(nest.strides[o][i]);
  }
  return FL_OK;
}

template <int VEC>
struct VecF {
  float v[VEC];
};

template <int VEC>
__device__ __forceinline__ VecF<VEC> LoadVec(const float *p) {
  VecF<VEC> r;
  if constexpr (VEC == 4) {
    const floatx4 t = *reinterpret_cast<const floatx4 *>(p);
    r.v[0] = t.x;
    r.v[1] = t.y;
    r.v[2] = t.z;
    r.v[3] = t.w;
  } else {
    r.v[0] = *p;
  }
  return r;
}

// Cooperative load of a ROWS x COLS tile whose COLS run along the operand's
// fast dimension. Out-of-range parts read as 0.
template <int ROWS, int COLS, int VEC, int NT>
struct TileLoader {
  static constexpr int kVecsPerRow = COLS / VEC;
  static constexpr int kItems = ROWS * kVecsPerRow;
  static constexpr int kPerThread = (kItems + NT - 1) / NT;

  // `tid`: index of the calling thread among the NT threads that share the tile
  __device__ __forceinline__ static void Load(const float *g, int row_stride, int col_stride, int rows_valid,
                                              int cols_valid, VecF<VEC> (&regs)[kPerThread], int tid) {
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      const int item = tid + j * NT;
      const int row = item / kVecsPerRow, col = (item % kVecsPerRow) * VEC;
      if (item < kItems && row < rows_valid && col < cols_valid) {
        regs[j] = LoadVec<VEC>(g + row * row_stride + col * col_stride);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) regs[j].v[i] = 0.0f;
      }
    }
  }

  __device__ __forceinline__ static void Store(float *lds, int ld, const VecF<VEC> (&regs)[kPerThread], int tid) {
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      const int item = tid + j * NT;
      const int row = item / kVecsPerRow, col = (item % kVecsPerRow) * VEC;
      if (item < kItems) {
        if constexpr (VEC == 4) {
          floatx4 t = {regs[j].v[0], regs[j].v[1], regs[j].v[2], regs[j].v[3]};
          *reinterpret_cast<floatx4 *>(lds + row * ld + col) = t;
        } else {
          lds[row * ld + col] = regs[j].v[0];
        }
      }
    }
  }
};

// The same tile as bf16: VEC consecutive values of a row become VEC consecutive 16-bit words (`ld` in 16-bit words, a
// multiple of 4).
template <typename Loader, int VEC>
__device__ __forceinline__ void StoreTileBf16(uint16_t *lds, int ld, const VecF<VEC> (&regs)[Loader::kPerThread], int tid,
                                              int nt) {
#pragma unroll
  for (int j = 0; j < Loader::kPerThread; ++j) {
    const int item = tid + j * nt;
    const int row = item / Loader::kVecsPerRow, col = (item % Loader::kVecsPerRow) * VEC;
    if (item < Loader::kItems) {
      if constexpr (VEC == 4) {
        *reinterpret_cast<u32x2 *>(lds + row * ld + col) =
            u32x2{PackBf16(regs[j].v[0], regs[j].v[1]), PackBf16(regs[j].v[2], regs[j].v[3])};
      } else {
        lds[row * ld + col] = static_cast<uint16_t>(ToBf16(regs[j].v[0]));
      }
    }
  }
}

// Eight 16-bit words `stride` words apart, packed as the matrix instruction wants its 8 values of k.
__device__ __forceinline__ u32x4 Gather8(const uint16_t *at, int stride) {
  uint32_t h[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) h[e] = at[e * stride];
  return u32x4{h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16};
}

// LA: 0 = A tile kept [m][k] (A is k-contiguous), 1 = kept [k][m].
// LB: 0 = B tile kept [k][n] (B is n-contiguous), 1 = kept [n][k].
// CONV: 0 = plain contraction; 1 = B is the input of a convolution addressed through p.conv (LB must be 0), one
// scalar gather per element; 2 = the same with one 128-bit gather per four consecutive output pixels of a row
// (unit stride along W in the input and in the convolution, OW a multiple of 4).
// SPEC: the workgroup has a second set of waves that only moves tiles from global memory into LDS (producers)
// while the first set only feeds the matrix cores from LDS (consumers).  With one workgroup per compute unit
// the plain kernel leaves each SIMD idle while its single wave waits for loads, writes LDS or sits at the
// barrier; here the two roles overlap.
// DIRECT (> 0: the number of stages in the ring): WM x WN x KS waves with one 32x32 MFMA tile each, operands
// k- resp. n-contiguous.  Tiles go from global memory straight into LDS (global_load_lds_dwordx4: every lane names
// its own 16 global bytes, the wave's 64 pieces land in one contiguous KiB of LDS), no registers and no LDS stores
// in between, so the number of bytes in flight is bounded by LDS (160 KB), not by registers.  A stage holds the
// k range of one chunk (BK = 32 KS) as [32][32] sub-tiles: WM x KS of A ([m][k]) and KS x WN of B ([k][n]); wave
// (wm, wn, ks) multiplies A(wm, ks) with B(ks, wn).  The 16-byte groups of a row of A are stored permuted (group q
// of row m in place q ^ ((m + m / 8) % 8)) so that the 128-bit operand reads of lanes with consecutive m fall on
// different banks without padding, which the contiguous landing area rules out.
//   WM = WN = 1 (the waves only split K): a wave loads exactly the two sub-tiles it multiplies, so the K loop has no
//   workgroup barrier at all -- the wave waits for its own oldest stage (vmcnt), runs its 16 MFMAs and requests
//   the stage DIRECT - 1 ahead.
//   Otherwise the loads of a stage are dealt evenly to the waves and one barrier per stage separates "my loads
//   of stage t have landed" from "stage t is read"; the same barrier tells that stage t - 1 has been read by
//   everyone, so its place is requested again right behind it.
template <int BM, int BN, int BK, int WM, int WN, int KS, int LA, int LB, int VEC, int DEPTH, int CONV = 0,
          bool BF16 = false, bool SPEC = false, int EXTRA = 0, int DIRECT = 0>
__global__ __launch_bounds__(64 * WM *WN *KS *(SPEC ? 2 : 1)) void MatmulKernel(float *__restrict__ C_, const float *__restrict__ A,
                                                                const float *__restrict__ B_, MatmulArgs p) {
  float *__restrict__ C = C_;
  const float *__restrict__ B = B_;
  constexpr int NT = 64 * WM * WN * KS;
  constexpr int TM = BM / (32 * WM), TN = BN / (32 * WN);
  constexpr int KW = BK / KS;  // k extent one wave covers per chunk
  static_assert(KW % (BF16 ? 16 : 8) == 0, "a wave consumes k in groups of 8 (bf16: 16)");
  // bf16 tiles: row pitches in 16-bit words (the regions keep the fp32 tiles' sizes: half of each stays unused)
  constexpr int LDAH = (LA == 0 ? BK : BM) + 8, LDBH = (LB == 0 ? BN : BK) + 8;

  constexpr int LDA = LA == 0 ? BK + 4 : BM;
  constexpr int LDB = LB == 0 ? BN : BK + 4;
  constexpr int A_ELEMS = LA == 0 ? BM * LDA : BK * LDA;
  constexpr int B_ELEMS = LB == 0 ? BK * LDB : BN * LDB;
  // QUARTER: one 32x32 tile per workgroup whose four waves split K.  After the K loop every wave takes a quarter of
  // the tile (8 rows: 4 of its 16 accumulator values per lane) through the rest of the kernel -- the sum over the
  // K slices, the exchange with the other K splits, bias, elementwise chain and stores -- instead of one wave
  // doing all 16 values while three have left.
  constexpr bool QUARTER = KS == 4 && TM * TN == 1 && WM * WN == 1;
  constexpr int EV = QUARTER ? 4 : 16;  // values per lane in the tail
  constexpr int RED_ELEMS = KS > 1 ? (QUARTER ? KS : KS - 1) * BM * BN : 0;
  constexpr int kSubTile = 1024;                            // floats of a [32][32] sub-tile (DIRECT)
  constexpr int kRingStage = (WM + WN) * KS * kSubTile;     // floats per stage of the ring (DIRECT)
  constexpr int kStageLoads = 4 * (WM + WN) * KS / (WM * WN * KS);  // load instructions per wave and stage (DIRECT)
  static_assert(DIRECT == 0 || (TM * TN == 1 && BK == 32 * KS && LA == 0 && LB == 0 && VEC == 4 && CONV == 0 && !SPEC &&
                                !BF16 && EXTRA != 2 && (4 * (WM + WN)) % (WM * WN) == 0 &&
                                kStageLoads * (DIRECT - 1) < 64),
                "the direct-to-LDS loop exists for one MFMA tile per wave of plain fp32 contractions");
  constexpr int STAGE_ELEMS = DIRECT > 0 ? DIRECT * kRingStage : 2 * (A_ELEMS + B_ELEMS);
  constexpr int LDS_ELEMS = STAGE_ELEMS > RED_ELEMS ? STAGE_ELEMS : RED_ELEMS;
  // (one LDS object per kernel: the row statistics of a deferred LayerNormalization live behind the tiles)
  constexpr int LN_ELEMS = EXTRA == 1 ? 2 * BM : 0;
  __shared__ __attribute__((aligned(16))) float lds[LDS_ELEMS + LN_ELEMS];

  // VEC: floats per global load of both operands' tiles; 41 = four for A and one for B (rows of B that do not keep
  // 16-byte alignment, a 7x7 image's 49 pixels, under weights that do)
  constexpr int VA = VEC == 41 ? 4 : VEC;
  constexpr int VB = CONV == 2 ? 4 : CONV == 1 || VEC == 41 ? 1 : VEC;
  // bf16: a B tile that arrives n-contiguous in 128-bit pieces is kept as [k / 2][n][2]: a thread stages the rows 2r
  // and 2r + 1 of its four columns, which are 16 consecutive bytes there, and the 8 values of k a lane feeds the
  // matrix instruction are four 32-bit words one pair-row apart (`LDPB` 16-bit words) -- no 16-bit accesses, no packing.
  constexpr bool PAIRED_B = BF16 && LB == 0 && VB == 4 && (BK * BN / 4 / NT) % 2 == 0 && BK * BN / 4 >= 2 * NT;
  constexpr int LDPB = 2 * BN + 16;
  // row of the B tile that item j of a thread stages, and the item's index among the tile's column groups
  auto b_item = [&](int j, int tid, int &row, int &colgroup) {
    constexpr int kGroups = BN / VB;
    if constexpr (PAIRED_B) {
      const int it = tid + (j / 2) * NT;
      row = 2 * (it / kGroups) + (j % 2);
      colgroup = it % kGroups;
    } else {
      const int it = tid + j * NT;
      row = it / kGroups;
      colgroup = it % kGroups;
    }
  };
  static_assert(!CONV || (LB == 0 && NT % (BN / VB) == 0), "the gather keeps one output pixel (group) per thread");
  static_assert(!SPEC || !CONV, "the gather of the convolution runs in the consumer waves");
  // EXTRA: 0 = none, 1 = addends in the epilogue, 2 = addends and a scale per row of B
  static_assert(EXTRA == 0 || (LB == 0 && CONV == 0), "the extra operands exist for plain contractions with B kept [k][n]");
  const bool producer = SPEC && threadIdx.x >= NT;
  const int ltid = producer ? static_cast<int>(threadIdx.x) - NT : static_cast<int>(threadIdx.x);
  using LoaderA = typename std::conditional<LA == 0, TileLoader<BM, BK, VA, NT>, TileLoader<BK, BM, VA, NT>>::type;
  using LoaderB = typename std::conditional<LB == 0, TileLoader<BK, BN, VB, NT>, TileLoader<BN, BK, VB, NT>>::type;

  // Request every argument the kernel is going to read in one batch and wait for them once: left to itself the
  // compiler loads each field right before its first use, a dozen dependent round trips to the scalar cache
  // before the first tile load can be issued.
  asm volatile("" ::"s"(p.M), "s"(p.N), "s"(p.K), "s"(p.sAm), "s"(p.sAk), "s"(p.sBk), "s"(p.sBn), "s"(p.sCm), "s"(p.sCn),
               "s"(p.tiles_m), "s"(p.tiles_n), "s"(p.n_splits), "s"(p.chunks_per_split), "s"(p.n_groups), "s"(p.n_inner),
               "s"(p.sCn_outer), "s"(p.bias), "s"(p.sDm), "s"(p.sDn), "s"(p.ca), "s"(p.cb), "s"(p.partials),
               "s"(p.counters), "s"(p.batch_rank), "s"(p.chain_n));
  if constexpr (EXTRA != 0) asm volatile("" ::"s"(p.addend), "s"(p.addend2), "s"(p.k_scale), "s"(p.sKs), "s"(p.addend_is_factor));
  if constexpr (EXTRA == 1) {
    asm volatile("" ::"s"(p.ln_mode), "s"(p.ln_parts), "s"(p.ln_width), "s"(p.ln_eps), "s"(p.ln_inv_width), "s"(p.ln_stats), "s"(p.ln_c1),
                 "s"(p.ln_scale), "s"(p.ln_shift), "s"(p.ln_s_scale), "s"(p.ln_s_shift), "s"(p.ln_s_c1), "s"(p.ln_stats_out));
  }
  if constexpr (CONV != 0) {
    asm volatile("" ::"s"(p.conv.H), "s"(p.conv.W), "s"(p.conv.sh), "s"(p.conv.sw), "s"(p.conv.dh), "s"(p.conv.dw),
                 "s"(p.conv.ph), "s"(p.conv.pw), "s"(p.conv.sXn), "s"(p.conv.sXc), "s"(p.conv.sXh), "s"(p.conv.sXw),
                 "s"(p.conv.sOn), "s"(p.conv.sOh), "s"(p.conv.sOw), "s"(p.conv.div_ohw.divisor),
                 "s"(p.conv.div_ohw.multiplier), "s"(p.conv.div_ohw.shift), "s"(p.conv.div_ow.divisor),
                 "s"(p.conv.div_ow.multiplier), "s"(p.conv.div_ow.shift), "s"(p.conv.div_khw.divisor),
                 "s"(p.conv.div_khw.multiplier), "s"(p.conv.div_khw.shift), "s"(p.conv.div_kw.divisor),
                 "s"(p.conv.div_kw.multiplier), "s"(p.conv.div_kw.shift));
  }

  // ---- which tile -----------------------------------------------------------
  uint32_t bid = blockIdx.x;
  const uint32_t n_tiles = p.tiles_m * p.tiles_n;
  if (n_tiles % 8 == 0) {
    // ids are dealt round-robin to the 8 XCDs: give each XCD a contiguous run
    bid = (bid % 8) * (n_tiles / 8) + bid / 8;
  }
  const int tile_m = bid % p.tiles_m, tile_n = bid / p.tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // which sibling of a grouped launch this workgroup serves
  const float *bias = p.bias;
  int32_t sCm = p.sCm, sCn = p.sCn, sCn_outer = p.sCn_outer;
  uint32_t batch_id = blockIdx.y;
  if (p.n_groups > 1) {
    if (batch_id > 0) {
      const uint32_t g = batch_id - 1;
      B = p.gB[g];
      C = p.gC[g];
      bias = p.gbias[g];
      sCm = p.g_sCm[g];
      sCn = p.g_sCn[g];
      sCn_outer = p.g_sCn_outer[g];
    }
    batch_id = 0;
  }
  int32_t boff[3] = {0, 0, 0};
  if (p.batch_rank > 0) {
    uint32_t rem = batch_id;
#pragma unroll
    for (int d = kMaxBatchDims - 1; d > 0; --d) {
      if (d < p.batch.rank) {
        uint32_t q, r;
        p.batch.div[d].DivMod(rem, q, r);
        rem = q;
#pragma unroll
        for (int o = 0; o < 3; ++o) boff[o] += static_cast<int32_t>(r) * p.batch.strides[o][d];
      }
    }
#pragma unroll
    for (int o = 0; o < 3; ++o) boff[o] += static_cast<int32_t>(rem) * p.batch.strides[o][0];
  }
  const float *Ab = A + boff[1] + static_cast<int64_t>(m0) * p.sAm;
  const float *Bb = CONV ? B : B + boff[2] + static_cast<int64_t>(n0) * p.sBn;
  float *Cb = C + boff[0];

  const int wave = ltid / 64, lane = threadIdx.x % 64;
  const int ks = wave % KS, wn = (wave / KS) % WN, wm = wave / (KS * WN);
  const int lrow = lane % 32, half = lane / 32;
  const int rows_m = p.M - m0, cols_n = p.N - n0;
  const int n_chunks = (p.K + BK - 1) / BK;
  // this workgroup's share of the chunks (all of them unless K is split over blockIdx.z)
  const int c_begin = p.n_splits > 1 ? static_cast<int>(blockIdx.z) * p.chunks_per_split : 0;
  const int c_end = p.n_splits > 1 ? min(n_chunks, c_begin + p.chunks_per_split) : n_chunks;

  // ---- direct loop: the first tile loads leave before anything else is asked of memory -------------------
  // (bias, addends, row statistics: a few hundred instructions of set-up that would otherwise stand between the
  // start of the wave and its first tile load)
  constexpr int R = DIRECT > 0 ? DIRECT : 1;
  constexpr bool PRIVATE = WM * WN == 1;  // every wave loads only what it reads itself
  const int n_st = c_end - c_begin;
  const int lr8 = lane / 8, lg = lane % 8;
  // This wave's loads of a stage: load i fills quarter j (rows 8j .. 8j+7) of sub-tile `sub`.  Per lane one global
  // pointer for the first stage and one step per stage; rows of A past M repeat the last row, columns of B past N
  // the first column group (their products are never stored).
  const float *gp[kStageLoads];
  int64_t step[kStageLoads];
  int32_t dst[kStageLoads];  // float offset inside the stage
#pragma unroll
  for (int i = 0; i < (DIRECT > 0 ? kStageLoads : 0); ++i) {
    const int q = PRIVATE ? (i < 4 ? 4 * wave + i : 4 * KS + 4 * wave + (i - 4)) : wave * kStageLoads + i;
    const int sub = q / 4, j = q % 4;
    dst[i] = q * 256;
    if (sub < WM * KS) {
      const int swm = sub / KS, sks = sub % KS;
      const int r = min(32 * swm + 8 * j + lr8, rows_m - 1);
      gp[i] = Ab + static_cast<int64_t>(r) * p.sAm + (c_begin * BK + sks * 32 + 4 * (lg ^ ((lr8 + j) & 7)));
      step[i] = BK;
    } else {
      const int sks = (sub - WM * KS) / WN, swn = (sub - WM * KS) % WN;
      const int col = 32 * swn + 4 * lg;
      gp[i] = Bb + static_cast<int64_t>(c_begin * BK + sks * 32 + 8 * j + lr8) * p.sBk + (col < cols_n ? col : -n0);
      step[i] = static_cast<int64_t>(BK) * p.sBk;
    }
  }
  float *ring = lds;
  auto issue = [&](int t, int slot) {
    float *at = ring + slot * kRingStage;
#pragma unroll
    for (int i = 0; i < kStageLoads; ++i) {
      // (operands copied into locals first: with an array element written directly as an argument of this
      // builtin the host pass silently drops the kernel's launch stub)
      const float *from = gp[i] + t * step[i];
      const int32_t to = dst[i];
      __builtin_amdgcn_global_load_lds(from, at + to, 16, 0, 0);
    }
  };
  // loads complete in order: "at most kStageLoads * later outstanding" means this wave's loads of stage t landed
  auto wait_for = [&](int later) {
    StaticFor<R>([&](auto n) {
      if (later == decltype(n)::value) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kStageLoads * decltype(n)::value) : "memory");
      }
    });
  };
  if constexpr (DIRECT > 0) {
#pragma unroll
    for (int s = 0; s < R - 1; ++s) {
      if (s < n_st) issue(s, s);
    }
  }

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // A bias with one value per column is requested now: at the end of the kernel its load would be one more
  // cold miss in the chain.
  const bool bias_by_col = bias != nullptr && p.sDm == 0;
  float bias_col[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + (wn * TN + j) * 32 + lrow;
    bias_col[j] = bias_by_col && n < p.N ? bias[n * p.sDn] : 0.0f;
  }

  // So are the tensors added after the chain, where a lane finishes few enough values (the quartered tail: the
  // four it will store).  Only the consumer waves of the last K split use them; the others' loads are dropped.
  constexpr bool PRE_ADD = EXTRA != 0 && QUARTER;
  float pre_add[PRE_ADD ? EV : 1], pre_add2[PRE_ADD ? EV : 1];
  if constexpr (PRE_ADD) {
    const int n = n0 + lrow;
#pragma unroll
    for (int e = 0; e < EV; ++e) {
      const int m = m0 + ks * 8 + half * 4 + e;
      const bool inside = !producer && m < p.M && n < p.N;
      const int64_t at = boff[0] + static_cast<int64_t>(m) * sCm + static_cast<int64_t>(n) * sCn;
      pre_add[e] = p.addend != nullptr && inside ? p.addend[at] : 0.0f;
      pre_add2[e] = p.addend2 != nullptr && inside ? p.addend2[at] : 0.0f;
    }
  }

  // Deferred LayerNormalization: the partial statistics of this workgroup's rows are requested now (NT / BM lanes
  // per row, each a few of the row's partials) and merged after the K loop, when they have long arrived.
  constexpr bool NORM = EXTRA == 1;
  constexpr int kNormLanes = NORM ? (NT / BM > 32 ? 32 : NT / BM) : 1;  // lanes per row, a power of two
  static_assert((kNormLanes & (kNormLanes - 1)) == 0, "the merge across a row's lanes is a butterfly");
  float *const ln_rows = lds + LDS_ELEMS;  // mean, then 1 / sqrt(var + eps), per row of the tile
  constexpr int kNormPer = 8;  // partials per lane: rows of up to 32 * kNormPer * kNormLanes elements
  float ln_part_mean[NORM ? kNormPer : 1], ln_part_m2[NORM ? kNormPer : 1];
  if constexpr (NORM) {
    if (p.ln_mode != 0 && !producer && ltid < BM * kNormLanes) {
      const int row = ltid / kNormLanes, sub = ltid % kNormLanes;
      const int m = min(m0 + row, p.M - 1);
#pragma unroll
      for (int u = 0; u < kNormPer; ++u) {
        const int q = sub + u * kNormLanes;
        const float *e = p.ln_stats + (static_cast<int64_t>(m) * p.ln_parts + min(q, p.ln_parts - 1)) * 2;
        ln_part_mean[u] = e[0];
        ln_part_m2[u] = e[1];
      }
    }
  }
  float ln_col[TN], ln_col2[TN];  // mode 1: c1 of the lane's columns; mode 2: scale and shift
  if constexpr (NORM) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + (wn * TN + j) * 32 + lrow;
      ln_col[j] = ln_col2[j] = 0.0f;
      if (p.ln_mode == 1 && n < p.N) {
        const float *c1 = blockIdx.y > 0 && p.n_groups > 1 ? p.g_ln_c1[blockIdx.y - 1] : p.ln_c1;
        ln_col[j] = c1[n * p.ln_s_c1];
      } else if (p.ln_mode == 2 && n < p.N) {
        ln_col[j] = p.ln_scale[n * p.ln_s_scale];
        ln_col2[j] = p.ln_shift[n * p.ln_s_shift];
      }
    }
  }

  // Called once the first tile loads are on their way: the statistics were requested before them and arrive first,
  // so the merge runs while the tiles travel; the barrier behind the K loop publishes its result.
  auto merge_rows = [&]() {
    if constexpr (NORM) {
      // Merge the row's partial statistics and leave mean and 1 / sqrt(var + eps) where the epilogue finds them.  Two
      // short passes without a division per partial: the mean of the row is the weighted mean of the partial means,
      // and the sum of squared deviations about it is the partials' own plus count * (partial mean - mean)^2 each --
      // deviations throughout, never a difference of large squares.
      if (p.ln_mode != 0 && !producer && ltid < BM * kNormLanes) {
        const int row = ltid / kNormLanes, sub = ltid % kNormLanes;
        float cnt[kNormPer];
        float sum = 0.0f;
#pragma unroll
        for (int u = 0; u < kNormPer; ++u) {
          const int q = sub + u * kNormLanes;
          cnt[u] = q < p.ln_parts ? static_cast<float>(min(32, p.ln_width - 32 * q)) : 0.0f;  // (absent: a clamped load)
          sum += cnt[u] * ln_part_mean[u];
        }
        const float mean = GroupSum<kNormLanes>(sum) * p.ln_inv_width;
        float m2 = 0.0f;
#pragma unroll
        for (int u = 0; u < kNormPer; ++u) {
          const float d = ln_part_mean[u] - mean;
          m2 += cnt[u] > 0.0f ? ln_part_m2[u] + cnt[u] * d * d : 0.0f;
        }
        m2 = GroupSum<kNormLanes>(m2);
        if (sub == 0) {
          ln_rows[row] = mean;
          ln_rows[BM + row] = 1.0f / sqrtf(m2 * p.ln_inv_width + p.ln_eps);
        }
      }
    }
  };

  // DEPTH chunks are in flight in registers: the loads of chunk c+DEPTH are issued while chunk c is
  // consumed, so a workgroup keeps DEPTH * (A tile + B tile) bytes outstanding instead of one chunk --
  // with only a few workgroups per CU that is what hides the L2/HBM latency.
  static_assert(DEPTH % 2 == 0, "the LDS buffer index must be a compile-time function of the stage");
  VecF<VA> ra[DEPTH][LoaderA::kPerThread];
  VecF<VB> rb[DEPTH][LoaderB::kPerThread];
  float rs[DEPTH][LoaderB::kPerThread];  // EXTRA == 2: the scale of the row each item of the B tile belongs to

  // convolution: the output pixel this thread gathers for stays the same for the whole kernel
  bool g_valid = false;
  int32_t g_ih0 = 0, g_iw0 = 0, g_base = 0;
  if constexpr (CONV) {
    const int n = n0 + static_cast<int>(threadIdx.x % (BN / VB)) * VB;
    g_valid = n < p.N;
    uint32_t img, r, oh, ow;
    p.conv.div_ohw.DivMod(static_cast<uint32_t>(g_valid ? n : 0), img, r);
    p.conv.div_ow.DivMod(r, oh, ow);
    g_ih0 = static_cast<int32_t>(oh) * p.conv.sh - p.conv.ph;
    g_iw0 = static_cast<int32_t>(ow) * p.conv.sw - p.conv.pw;
    g_base = static_cast<int32_t>(img) * p.conv.sXn;
  }

  auto load_chunk = [&](int c, VecF<VA>(&qa)[LoaderA::kPerThread], VecF<VB>(&qb)[LoaderB::kPerThread],
                        float(&qs)[LoaderB::kPerThread]) {
    const int k0 = c * BK, k_valid = p.K - k0;
    if constexpr (EXTRA == 2) {
      if (p.k_scale != nullptr) {
#pragma unroll
        for (int j = 0; j < LoaderB::kPerThread; ++j) {
          const int k = k0 + (ltid + j * NT) / LoaderB::kVecsPerRow;
          qs[j] = k < p.K ? p.k_scale[static_cast<int64_t>(k) * p.sKs] : 0.0f;
        }
      }
    }
    if constexpr (LA == 0) {
      LoaderA::Load(Ab + static_cast<int64_t>(k0) * p.sAk, p.sAm, p.sAk, rows_m, k_valid, qa, ltid);
    } else {
      LoaderA::Load(Ab + static_cast<int64_t>(k0) * p.sAk, p.sAk, p.sAm, k_valid, rows_m, qa, ltid);
    }
    if constexpr (CONV) {
      // same item -> (k row, n column) mapping as TileLoader<BK, BN, VB, NT>: column group = thread % (BN / VB)
#pragma unroll
      for (int j = 0; j < LoaderB::kPerThread; ++j) {
        int b_row, b_group;
        b_item(j, static_cast<int>(threadIdx.x), b_row, b_group);  // (the column group is this thread's for every j)
        const int k = k0 + b_row;
#pragma unroll
        for (int e = 0; e < VB; ++e) qb[j].v[e] = 0.0f;
        if (g_valid && k < p.K) {
          uint32_t ci, r, kh, kw;
          p.conv.div_khw.DivMod(static_cast<uint32_t>(k), ci, r);
          p.conv.div_kw.DivMod(r, kh, kw);
          const int32_t ih = g_ih0 + static_cast<int32_t>(kh) * p.conv.dh;
          const int32_t iw = g_iw0 + static_cast<int32_t>(kw) * p.conv.dw;
          if (static_cast<uint32_t>(ih) < static_cast<uint32_t>(p.conv.H)) {
            if constexpr (CONV == 2) {
              // four output pixels of one row read four consecutive input elements (4-byte aligned only)
              const float *row = B + g_base + static_cast<int32_t>(ci) * p.conv.sXc + ih * p.conv.sXh;
              if (iw >= 0 && iw + 3 < p.conv.W) {
                struct __attribute__((packed, aligned(4))) Quad {
                  float v[4];
                };
                const Quad q = *reinterpret_cast<const Quad *>(row + iw);
#pragma unroll
                for (int e = 0; e < 4; ++e) qb[j].v[e] = q.v[e];
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  if (static_cast<uint32_t>(iw + e) < static_cast<uint32_t>(p.conv.W)) qb[j].v[e] = row[iw + e];
                }
              }
            } else if (static_cast<uint32_t>(iw) < static_cast<uint32_t>(p.conv.W)) {
              qb[j].v[0] = B[g_base + static_cast<int32_t>(ci) * p.conv.sXc + ih * p.conv.sXh + iw * p.conv.sXw];
            }
          }
        }
      }
    } else if constexpr (PAIRED_B) {
#pragma unroll
      for (int j = 0; j < LoaderB::kPerThread; ++j) {
        int row, group;
        b_item(j, ltid, row, group);
        const int col = group * VB;
        if (row < k_valid && col < cols_n) {
          qb[j] = LoadVec<VB>(Bb + static_cast<int64_t>(k0 + row) * p.sBk + static_cast<int64_t>(col) * p.sBn);
        } else {
#pragma unroll
          for (int e = 0; e < VB; ++e) qb[j].v[e] = 0.0f;
        }
      }
    } else if constexpr (LB == 0) {
      LoaderB::Load(Bb + static_cast<int64_t>(k0) * p.sBk, p.sBk, p.sBn, k_valid, cols_n, qb, ltid);
    } else {
      LoaderB::Load(Bb + static_cast<int64_t>(k0) * p.sBk, p.sBn, p.sBk, cols_n, k_valid, qb, ltid);
    }
  };
  auto store_chunk = [&](int buf, const VecF<VA>(&qa)[LoaderA::kPerThread], const VecF<VB>(&qb)[LoaderB::kPerThread],
                         const float(&qs)[LoaderB::kPerThread]) {
    float *as = lds + buf * (A_ELEMS + B_ELEMS);
    float *bs = as + A_ELEMS;
    if constexpr (BF16) {
      StoreTileBf16<LoaderA, VA>(reinterpret_cast<uint16_t *>(as), LDAH, qa, ltid, NT);
      if constexpr (PAIRED_B) {
        uint16_t *bh = reinterpret_cast<uint16_t *>(bs);
#pragma unroll
        for (int j = 0; j < LoaderB::kPerThread; j += 2) {
          int row, group;
          b_item(j, ltid, row, group);
          *reinterpret_cast<u32x4 *>(bh + (row / 2) * LDPB + group * 8) =
              u32x4{PackBf16(qb[j].v[0], qb[j + 1].v[0]), PackBf16(qb[j].v[1], qb[j + 1].v[1]),
                    PackBf16(qb[j].v[2], qb[j + 1].v[2]), PackBf16(qb[j].v[3], qb[j + 1].v[3])};
        }
      } else {
        StoreTileBf16<LoaderB, VB>(reinterpret_cast<uint16_t *>(bs), LDBH, qb, ltid, NT);
      }
      return;
    }
    LoaderA::Store(as, LDA, qa, ltid);
    if constexpr (EXTRA == 2) {
      if (p.k_scale != nullptr) {
        VecF<VB> scaled[LoaderB::kPerThread];
#pragma unroll
        for (int j = 0; j < LoaderB::kPerThread; ++j)
#pragma unroll
          for (int e = 0; e < VB; ++e) scaled[j].v[e] = qb[j].v[e] * qs[j];
        LoaderB::Store(bs, LDB, scaled, ltid);
        return;
      }
    }
    LoaderB::Store(bs, LDB, qb, ltid);
  };
  auto compute_chunk = [&](int buf) {
    const float *as = lds + buf * (A_ELEMS + B_ELEMS);
    const float *bs = as + A_ELEMS;
    if constexpr (BF16) {
      const uint16_t *ah = reinterpret_cast<const uint16_t *>(as), *bh = reinterpret_cast<const uint16_t *>(bs);
#pragma unroll
      for (int kk = 0; kk < KW; kk += 16) {
        const int k8 = ks * KW + kk + 8 * half;
        u32x4 a8[TM], b8[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int m = (wm * TM + i) * 32 + lrow;
          if constexpr (LA == 0) a8[i] = *reinterpret_cast<const u32x4 *>(ah + m * LDAH + k8);
          else a8[i] = Gather8(ah + k8 * LDAH + m, LDAH);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int n = (wn * TN + j) * 32 + lrow;
          if constexpr (PAIRED_B) {
            const uint32_t *w = reinterpret_cast<const uint32_t *>(bh + (k8 / 2) * LDPB) + n;
            b8[j] = u32x4{w[0], w[LDPB / 2], w[2 * (LDPB / 2)], w[3 * (LDPB / 2)]};
          } else if constexpr (LB == 0) {
            b8[j] = Gather8(bh + k8 * LDBH + n, LDBH);
          } else {
            b8[j] = *reinterpret_cast<const u32x4 *>(bh + n * LDBH + k8);
          }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a8[i]), __builtin_bit_cast(bf16x8, b8[j]),
                                                                acc[i][j], 0, 0, 0);
      }
      return;
    }
#pragma unroll
    for (int kk = 0; kk < KW; kk += 8) {
      const int kbase = ks * KW + kk + 4 * half;
      float a[TM][4], b[TN][4];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int m = (wm * TM + i) * 32 + lrow;
        if constexpr (LA == 0) {
          const floatx4 t = *reinterpret_cast<const floatx4 *>(as + m * LDA + kbase);
          a[i][0] = t.x;
          a[i][1] = t.y;
          a[i][2] = t.z;
          a[i][3] = t.w;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) a[i][e] = as[(kbase + e) * LDA + m];
        }
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = (wn * TN + j) * 32 + lrow;
        if constexpr (LB == 0) {
#pragma unroll
          for (int e = 0; e < 4; ++e) b[j][e] = bs[(kbase + e) * LDB + n];
        } else {
          const floatx4 t = *reinterpret_cast<const floatx4 *>(bs + n * LDB + kbase);
          b[j][0] = t.x;
          b[j][1] = t.y;
          b[j][2] = t.z;
          b[j][3] = t.w;
        }
      }
      {
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][e], b[j][e], acc[i][j], 0, 0, 0);
      }
    }
  };

  if constexpr (DIRECT > 0) {
    const int sw = (lrow + (lrow >> 3)) & 7;
    const int a_sub = (wm * KS + ks) * kSubTile, b_sub = (WM * KS + ks * WN + wn) * kSubTile;
    merge_rows();
    // Stage t, held in place `slot` (t % R, a constant so that the LDS offsets are immediates).
    auto stage = [&](int t, auto slot_c) {
      constexpr int slot = decltype(slot_c)::value;
      // Place (slot + R - 1) % R held stage t - 1.  PRIVATE: this wave's reads of it have returned (the MFMAs that
      // use them are issued).  Shared: every wave passed this stage's barrier only after reading stage t - 1.
      if constexpr (PRIVATE) {
        if (t + R - 1 < n_st) issue(t + R - 1, (slot + R - 1) % R);
        wait_for(min(n_st - 1, t + R - 1) - t);
      } else {
        wait_for(min(n_st - 1, t + R - 2) - t);
        // (the bare barrier: __syncthreads() adds a fence that waits for every outstanding load, the stages
        // in flight included; all that has to be ordered here are the tile loads, waited for just above, and
        // the LDS reads of stage t - 1, which returned before their MFMAs were issued)
        __builtin_amdgcn_s_barrier();
        if (t + R - 1 < n_st) issue(t + R - 1, (slot + R - 1) % R);
      }
      const float *as = lds + slot * kRingStage + a_sub;
      const float *bs = lds + slot * kRingStage + b_sub;
      // all of the stage's operands are requested before the first product, so that the LDS round trips overlap
      floatx4 a4[4];
      float b4[4][4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        a4[q] = *reinterpret_cast<const floatx4 *>(as + lrow * 32 + 4 * ((2 * q + half) ^ sw));
#pragma unroll
        for (int e = 0; e < 4; ++e) b4[q][e] = bs[(8 * q + 4 * half + e) * 32 + lrow];
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[q].x, b4[q][0], acc[0][0], 0, 0, 0);
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[q].y, b4[q][1], acc[0][0], 0, 0, 0);
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[q].z, b4[q][2], acc[0][0], 0, 0, 0);
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[q].w, b4[q][3], acc[0][0], 0, 0, 0);
      }
    };
    // Whole rounds of the ring run without a condition around the products: with one, the compiler carries the
    // accumulator through the loop in vector registers and moves all 16 to the accumulation registers and back
    // around every stage.  The last n_st % R stages follow.
    int t0 = 0;
    for (; t0 + R <= n_st; t0 += R) {
      StaticFor<R>([&](auto slot_c) { stage(t0 + decltype(slot_c)::value, slot_c); });
    }
    StaticFor<R - 1>([&](auto slot_c) {
      if (t0 + decltype(slot_c)::value < n_st) stage(t0 + decltype(slot_c)::value, slot_c);  // uniform over the workgroup
    });
  } else if constexpr (SPEC) {
    // Barrier j separates "chunk j is in LDS" from "chunk j is being consumed".  Producers store chunk j after
    // barrier j-1 (the consumers are then done with chunk j-2, the previous content of that buffer); consumers
    // compute chunk j after barrier j.  Both sides pass one barrier per chunk.
    if (!producer) merge_rows();
    if (producer) {
#pragma unroll
      for (int s = 0; s < DEPTH; ++s) {
        if (c_begin + s < c_end) load_chunk(c_begin + s, ra[s], rb[s], rs[s]);
      }
      for (int c0 = c_begin; c0 < c_end; c0 += DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; ++s) {
          const int c = c0 + s;
          if (c < c_end) {  // uniform over the workgroup
            if (c > c_begin) __syncthreads();
            store_chunk(s & 1, ra[s], rb[s], rs[s]);
            if (c + DEPTH < c_end) load_chunk(c + DEPTH, ra[s], rb[s], rs[s]);
          }
        }
      }
      __syncthreads();  // the last chunk is in LDS
    } else {
      for (int c0 = c_begin; c0 < c_end; c0 += DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; ++s) {
          if (c0 + s < c_end) {
            __syncthreads();
            compute_chunk(s & 1);
          }
        }
      }
    }
  } else {
#pragma unroll
    for (int s = 0; s < DEPTH; ++s) {
      if (c_begin + s < c_end) load_chunk(c_begin + s, ra[s], rb[s], rs[s]);
    }
    merge_rows();
    for (int c0 = c_begin; c0 < c_end; c0 += DEPTH) {
#pragma unroll
      for (int s = 0; s < DEPTH; ++s) {
        const int c = c0 + s;
        if (c < c_end) {  // uniform over the workgroup
          store_chunk(s & 1, ra[s], rb[s], rs[s]);
          if (c + DEPTH < c_end) load_chunk(c + DEPTH, ra[s], rb[s], rs[s]);
          // one barrier per chunk: buffer (s&1) was last read two chunks ago, and every wave
          // passed the previous barrier only after finishing that read
          __syncthreads();
          compute_chunk(s & 1);
        }
      }
    }
  }
  __syncthreads();  // staging area is reused below

  // ---- combine the K slices of a workgroup through LDS ------------------------
  if constexpr (QUARTER) {
    if (!producer) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        lds[ks * BM * BN + ((e / 4) * 8 + half * 4 + (e % 4)) * BN + lrow] = acc[0][0][e];
      }
    }
    __syncthreads();
    if (producer) return;
    // value i of the quarter is accumulator element 4 ks + i: tile row 8 ks + 4 half + i; slices added in order
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int at = (ks * 8 + half * 4 + i) * BN + lrow;
      acc[0][0][i] = ((lds[at] + lds[BM * BN + at]) + lds[2 * BM * BN + at]) + lds[3 * BM * BN + at];
    }
  } else if constexpr (KS > 1) {
    if (ks > 0 && !producer) {
      float *red = lds + (ks - 1) * BM * BN;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int m = (wm * TM + i) * 32 + (e / 4) * 8 + half * 4 + (e % 4);
            const int n = (wn * TN + j) * 32 + lrow;
            red[m * BN + n] = acc[i][j][e];
          }
    }
    __syncthreads();
    if (ks > 0 || producer) return;
#pragma unroll
    for (int s = 1; s < KS; ++s) {
      const float *red = lds + (s - 1) * BM * BN;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int m = (wm * TM + i) * 32 + (e / 4) * 8 + half * 4 + (e % 4);
            const int n = (wn * TN + j) * 32 + lrow;
            acc[i][j][e] += red[m * BN + n];
          }
    }
  }

  if (producer) return;

  // ---- combine the K splits of a tile across workgroups ------------------------
  // Only configurations in which a wave ends up with exactly one 32x32 accumulator split (host side), and each
  // wave runs the protocol on its own slot, so no workgroup barrier is involved: the wave publishes its partial
  // tile, then one atomic tells it whether it arrived last; the last wave adds all partials in split order,
  // which makes the sum independent of arrival order.
  if constexpr (TM * TN == 1 && (WM * WN == 1 || KS == 1 || DIRECT > 0)) {
    if (p.n_splits > 1) {
      const uint32_t n_splits = p.n_splits;
      const uint32_t tile_id = (blockIdx.y * n_tiles + blockIdx.x) * (WM * WN) + wm * WN + wn;
      // a wave's slot: the whole tile, or its quarter of it (own arrival counter per quarter)
      const uint32_t slot = QUARTER ? tile_id * 4 + ks : tile_id;
      const uint32_t sub = QUARTER ? ks * 256 : 0;
      float *mine = p.partials + (static_cast<size_t>(tile_id) * n_splits + blockIdx.z) * 1024 + sub;
      // The partial tiles travel through device-coherent accesses (agent-scope atomics: write-through stores
      // and loads that miss in the per-XCD L2), so no cache-wide write-back or invalidate is needed.
      // Release side: a fence of workgroup scope emits no wait on this target (the L1 keeps one workgroup's
      // accesses in order), and the stores and the counter go to different L2 channels, so the wave itself
      // waits until every vector memory operation it has issued is acknowledged (s_waitcnt vmcnt(0); stores
      // count in vmcnt on gfx9) before it counts its arrival.  The "memory" clobber keeps the compiler from
      // moving the stores below the wait or the counter update above it.
      // Acquire side: the partial loads are issued after the branch on the counter's returned value, which
      // the wave has to wait for; the compiler-only fence below keeps them behind it in program order.
#pragma unroll
      for (int e = 0; e < EV; ++e) {
        __hip_atomic_store(mine + e * 64 + lane, acc[0][0][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      uint32_t arrived = 0;
      if (lane == 0) arrived = __hip_atomic_fetch_add(&p.counters[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      arrived = __shfl(arrived, 0);
      if (arrived != n_splits - 1) return;
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // compiler ordering only: no instruction on gfx9
      if (lane == 0) __hip_atomic_store(&p.counters[slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const float *all = p.partials + static_cast<size_t>(tile_id) * n_splits * 1024 + sub;
#pragma unroll
      for (int e = 0; e < EV; ++e) acc[0][0][e] = 0.0f;
      // four splits' loads are in flight together (one round trip for up to four splits); the sums still run
      // in split order
      for (uint32_t z0 = 0; z0 < n_splits; z0 += 4) {
        float part[4][EV];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
          const uint32_t z = z0 + u < n_splits ? z0 + u : z0;  // repeats a valid slot, ignored below
#pragma unroll
          for (int e = 0; e < EV; ++e) {
            part[u][e] = __hip_atomic_load(all + z * 1024 + e * 64 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
          if (z0 + u < n_splits) {
#pragma unroll
            for (int e = 0; e < EV; ++e) acc[0][0][e] += part[u][e];
          }
        }
      }
    }
  }

  // ---- epilogue ---------------------------------------------------------------
  StaticFor<TM * TN>([&](auto tile) {
      constexpr int i = decltype(tile)::value / TN, j = decltype(tile)::value % TN;
      const int n = n0 + (wn * TN + j) * 32 + lrow;
      int64_t col = static_cast<int64_t>(n) * sCn;
      if (!CONV && p.n_inner != 0) {
        uint32_t hi, lo;
        p.div_inner.DivMod(static_cast<uint32_t>(n < p.N ? n : 0), hi, lo);
        col = static_cast<int64_t>(hi) * sCn_outer + static_cast<int64_t>(lo) * sCn;
      }
      if constexpr (CONV) {
        uint32_t img, r, oh, ow;
        p.conv.div_ohw.DivMod(static_cast<uint32_t>(n < p.N ? n : 0), img, r);
        p.conv.div_ow.DivMod(r, oh, ow);
        col = static_cast<int64_t>(img) * p.conv.sOn + static_cast<int64_t>(oh) * p.conv.sOh +
              static_cast<int64_t>(ow) * p.conv.sOw;
      }
      // bias, then the elementwise chain on the values of this 32x32 tile the lane holds (all 16, or the 4 of its
      // wave's quarter), then the stores
      auto tile_row = [&](int e) { return QUARTER ? ks * 8 + half * 4 + e : (e / 4) * 8 + half * 4 + (e % 4); };
      float vals[EV];
#pragma unroll
      for (int e = 0; e < EV; ++e) {
        const int m = m0 + (wm * TM + i) * 32 + tile_row(e);
        float v = acc[i][j][e];
        if constexpr (NORM) {
          if (p.ln_mode == 1) {
            // A was the un-normalised tensor: LayerNorm(t) . B = rstd * (t . (scale B) - mean * colsum(scale B)) + shift . B
            const int r = (wm * TM + i) * 32 + tile_row(e);
            v = ln_rows[BM + r] * (v - ln_rows[r] * ln_col[j]);
          }
        }
        if (bias_by_col) {
          v = p.ca * v + p.cb * bias_col[j];
        } else if (bias != nullptr && m < p.M && n < p.N) {
          v = p.ca * v + p.cb * bias[m * p.sDm + n * p.sDn];
        }
        vals[e] = v;
      }
      if (p.chain_n != 0) RunChainBlock<EV>(p.chain, vals);
      if constexpr (EXTRA != 0) {
        // both tensors are requested before either is added
        if (p.addend != nullptr) {
          const float *Eb = p.addend + boff[0], *Eb2 = p.addend2 != nullptr ? p.addend2 + boff[0] : nullptr;
          float add[EV], add2[EV];
#pragma unroll
          for (int e = 0; e < EV; ++e) {
            if constexpr (PRE_ADD) {
              add[e] = pre_add[e];
              add2[e] = pre_add2[e];
            } else {
              const int m = m0 + (wm * TM + i) * 32 + tile_row(e);
              const bool inside = m < p.M && n < p.N;
              add[e] = inside ? Eb[static_cast<int64_t>(m) * sCm + col] : 0.0f;
              add2[e] = Eb2 != nullptr && inside ? Eb2[static_cast<int64_t>(m) * sCm + col] : 0.0f;
            }
          }
          if constexpr (NORM) {
            if (p.ln_mode == 2) {
              // the addend is the un-normalised tensor of a LayerNormalization: normalise it on the way in
#pragma unroll
              for (int e = 0; e < EV; ++e) {
                const int r = (wm * TM + i) * 32 + tile_row(e);
                add[e] = (add[e] - ln_rows[r]) * ln_rows[BM + r] * ln_col[j] + ln_col2[j];
              }
            }
          }
          if (p.addend_is_factor != 0) {
#pragma unroll
            for (int e = 0; e < EV; ++e) vals[e] *= add[e];
          } else {
#pragma unroll
            for (int e = 0; e < EV; ++e) vals[e] += add[e];
          }
          if (Eb2 != nullptr) {
#pragma unroll
            for (int e = 0; e < EV; ++e) vals[e] += add2[e];
          }
        }
      }
#pragma unroll
      for (int e = 0; e < EV; ++e) {
        const int m = m0 + (wm * TM + i) * 32 + tile_row(e);
        if (m < p.M && n < p.N) Cb[static_cast<int64_t>(m) * sCm + col] = vals[e];
      }
      if constexpr (NORM) {
        if (p.ln_stats_out != nullptr) {
          // statistics of this 32-column run of every row the lane's half-wave holds: mean, then the sum of squared
          // deviations from it (two butterflies over the 32 lanes of the half; columns past N count as absent)
          const int first = n0 + (wn * TN + j) * 32;
          const float inv_cols = 1.0f / static_cast<float>(min(32, p.N - first));
          const int parts = (p.N + 31) / 32;
#pragma unroll
          for (int e = 0; e < EV; ++e) {
            const float mean = GroupSum<32>(n < p.N ? vals[e] : 0.0f) * inv_cols;
            const float d = n < p.N ? vals[e] - mean : 0.0f;
            const float sq = GroupSum<32>(d * d);
            const int m = m0 + (wm * TM + i) * 32 + tile_row(e);
            if (lrow == 0 && m < p.M && first < p.N) {
              float *at = p.ln_stats_out + (static_cast<int64_t>(m) * parts + first / 32) * 2;
              *reinterpret_cast<float2 *>(at) = make_float2(mean, sq);
            }
          }
        }
      }
  });
}

// ---- skinny contraction: M <= 8 rows against a k-contiguous B (weight streaming, HBM bound) ----------------
// One wave owns kSkinnyRows (1, 2 or 4: fewer when N alone cannot fill the chip) consecutive columns n of C, i.e. rows of B as stored: lanes stride K with 128-bit
// loads of those rows and of the M rows of A (small, served by the caches), keep M x kSkinnyRows partial sums
// each and combine them with wave64 shuffles.  No LDS, no MFMA: at one to eight rows the matrix cores would
// run 75-97 % empty while the kernel waits for the weights anyway.
template <int MT, int kSkinnyRows>
__global__ __launch_bounds__(256) void SkinnyGemmKernel(float *__restrict__ C, const float *__restrict__ A,
                                                        const float *__restrict__ B, MatmulArgs p) {
  const int lane = threadIdx.x % 64;
  const int n0 = (blockIdx.x * 4 + threadIdx.x / 64) * kSkinnyRows;
  if (n0 >= p.N) return;
  float acc[MT][kSkinnyRows];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < kSkinnyRows; ++r) acc[m][r] = 0.0f;
  const float *brow[kSkinnyRows];
#pragma unroll
  for (int r = 0; r < kSkinnyRows; ++r) brow[r] = B + static_cast<int64_t>(min(n0 + r, p.N - 1)) * p.sBn;
  // two 256-wide k steps per iteration: 2 x kSkinnyRows 128-bit weight loads in flight per lane
  for (int k = lane * 4; k < p.K; k += 512) {
    const bool second = k + 256 < p.K;
    floatx4 b0[kSkinnyRows], b1[kSkinnyRows], a0[MT], a1[MT];
#pragma unroll
    for (int r = 0; r < kSkinnyRows; ++r) {
      b0[r] = *reinterpret_cast<const floatx4 *>(brow[r] + k);
      b1[r] = second ? *reinterpret_cast<const floatx4 *>(brow[r] + k + 256) : floatx4{0, 0, 0, 0};
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const float *arow = A + static_cast<int64_t>(m) * p.sAm + k;
      a0[m] = m < p.M ? *reinterpret_cast<const floatx4 *>(arow) : floatx4{0, 0, 0, 0};
      a1[m] = m < p.M && second ? *reinterpret_cast<const floatx4 *>(arow + 256) : floatx4{0, 0, 0, 0};
    }
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < kSkinnyRows; ++r) {
        acc[m][r] += a0[m].x * b0[r].x;
        acc[m][r] += a0[m].y * b0[r].y;
        acc[m][r] += a0[m].z * b0[r].z;
        acc[m][r] += a0[m].w * b0[r].w;
        acc[m][r] += a1[m].x * b1[r].x;
        acc[m][r] += a1[m].y * b1[r].y;
        acc[m][r] += a1[m].z * b1[r].z;
        acc[m][r] += a1[m].w * b1[r].w;
      }
  }
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < kSkinnyRows; ++r) acc[m][r] = WaveReduce(acc[m][r], SumOp{});
  if (lane == 0) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < kSkinnyRows; ++r) {
        const int n = n0 + r;
        if (m < p.M && n < p.N) {
          float v = acc[m][r];
          if (p.bias != nullptr) v = p.ca * v + p.cb * p.bias[m * p.sDm + n * p.sDn];
          if (p.chain.n != 0) v = RunChain(p.chain, v);
          C[static_cast<int64_t>(m) * p.sCm + static_cast<int64_t>(n) * p.sCn] = v;
        }
      }
  }
}

// The same for long K (K >= 2048): a whole workgroup owns ROWS columns n of C and its four waves split K, so that four
// times as many waves stream weights at once (N = 4096, K = 25088: 8 waves per compute unit with the kernel above keep
// ~8 MB in flight, too little to cover the memory latency at the HBM rate); the four partial sums of every output are
// added in wave order through LDS.  Every workgroup reads all of A, whatever ROWS is: with M rows of A the caches
// deliver M / ROWS bytes of A per byte of weights, so ROWS grows with M (M = 8, ROWS = 2: 1.6 GB of A through L2 for
// 411 MB of weights, 129 us; the weights alone take 63 us at 6.5 TB/s).  STEPS k steps of 1024 per iteration.
template <int MT, int ROWS, int STEPS>
__global__ __launch_bounds__(256) void SkinnyGemmBlockKernel(float *__restrict__ C, const float *__restrict__ A,
                                                             const float *__restrict__ B, MatmulArgs p) {
  __shared__ float partial[4][MT][ROWS];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int n0 = blockIdx.x * ROWS;
  float acc[MT][ROWS];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[m][r] = 0.0f;
  const float *brow[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) brow[r] = B + static_cast<int64_t>(min(n0 + r, p.N - 1)) * p.sBn;
  for (int k = threadIdx.x * 4; k < p.K; k += 1024 * STEPS) {
    floatx4 b[STEPS][ROWS], a[STEPS][MT];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      const bool live = k + 1024 * t < p.K;
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        b[t][r] = live ? *reinterpret_cast<const floatx4 *>(brow[r] + k + 1024 * t) : floatx4{0, 0, 0, 0};
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const float *arow = A + static_cast<int64_t>(m) * p.sAm + k + 1024 * t;
        a[t][m] = m < p.M && live ? *reinterpret_cast<const floatx4 *>(arow) : floatx4{0, 0, 0, 0};
      }
    }
#pragma unroll
    for (int t = 0; t < STEPS; ++t)
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
          acc[m][r] += a[t][m].x * b[t][r].x;
          acc[m][r] += a[t][m].y * b[t][r].y;
          acc[m][r] += a[t][m].z * b[t][r].z;
          acc[m][r] += a[t][m].w * b[t][r].w;
        }
  }
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const float v = WaveReduce(acc[m][r], SumOp{});
      if (lane == 0) partial[wave][m][r] = v;
    }
  __syncthreads();
  if (threadIdx.x < MT * ROWS) {
    const int m = threadIdx.x / ROWS, r = threadIdx.x % ROWS, n = n0 + r;
    if (m < p.M && n < p.N) {
      float v = ((partial[0][m][r] + partial[1][m][r]) + partial[2][m][r]) + partial[3][m][r];
      if (p.bias != nullptr) v = p.ca * v + p.cb * p.bias[m * p.sDm + n * p.sDn];
      if (p.chain.n != 0) v = RunChain(p.chain, v);
      C[static_cast<int64_t>(m) * p.sCm + static_cast<int64_t>(n) * p.sCn] = v;
    }
  }
}

// Launches the skinny kernel if the problem fits it; false = use the tiled kernel.
inline bool TrySkinnyGemm(const MatmulArgs &p, int64_t n_batch, float *C, const float *A, const float *B, hipStream_t s) {
  if (n_batch != 1 || p.M > 8 || p.N < 256 || p.K < 256 || p.n_inner != 0 || p.n_groups > 1) return false;
  // Five to eight rows against many long weight rows: every lane of the kernels below loads M values of A per
  // weight value, and from five rows on those cache reads, not HBM, set the pace; the tiled kernel shares A through
  // LDS and splits K over workgroups ([8,25088] x [4096,25088]^T: 78.7 against 89.8 us, [8,4096] x [4096,4096]^T:
  // 17.3 against 21.6; with fewer weight rows or a shorter K it has too few tiles: [8,4096] x [1000,4096]^T 11.3
  // against 8.8 us).  A 16x16x4 MFMA formulation of the streaming kernel (16 weight rows per wave, both operands
  // loaded 128 bits along k) was measured as well: 91 us at eight rows.
  if (p.M >= 5 && p.N >= 2048 && p.K >= 2048) return false;
  if (p.sBk != 1 || p.sAk != 1 || p.K % 4 != 0 || p.sBn % 4 != 0 || (p.M > 1 && p.sAm % 4 != 0)) return false;
  if (!IsAligned(A, 16) || !IsAligned(B, 16)) return false;
  if (p.K >= 2048) {
    // columns per workgroup: as many as A has rows (at least two), while two workgroups per compute unit remain
    const int mt = p.M == 1 ? 1 : p.M == 2 ? 2 : p.M <= 4 ? 4 : 8;
    // (with K below 8192 a workgroup runs too few iterations for the wider variants to pay: 4096 x 4096 at M = 8
    // takes 24.7 us with two columns, 27.8 us with eight)
    int rows = p.K >= 8192 ? std::max(mt, 2) : 2;
    while (rows > 1 && p.N / rows < 512) rows /= 2;
    // (sixteen columns per workgroup at M = 8 -- half the re-reads of A -- were measured slower: 106 against 90.5 us for
    // [8,25088] x [4096,25088]^T; with 128 accumulators only four waves per compute unit stream weights)
#define FL_SKINNY_BLOCK(MT_, ROWS_)                                                                              \
  FL_LAUNCH((SkinnyGemmBlockKernel<MT_, ROWS_, (MT_ * ROWS_ <= 8 ? 2 : 1)>), dim3((p.N + ROWS_ - 1) / ROWS_), dim3(256), 0, \
            s, C, A, B, p)
#define FL_SKINNY_ROWS(MT_)                    \
  do {                                         \
    if (rows == 8) FL_SKINNY_BLOCK(MT_, 8);    \
    else if (rows == 4) FL_SKINNY_BLOCK(MT_, 4); \
    else if (rows == 2) FL_SKINNY_BLOCK(MT_, 2); \
    else FL_SKINNY_BLOCK(MT_, 1);              \
  } while (0)
    if (mt == 1) FL_SKINNY_ROWS(1);
    else if (mt == 2) FL_SKINNY_ROWS(2);
    else if (mt == 4) FL_SKINNY_ROWS(4);
    else FL_SKINNY_ROWS(8);
#undef FL_SKINNY_ROWS
#undef FL_SKINNY_BLOCK
    return true;
  }
  // rows per wave: as many as still leave about eight waves per compute unit
  const int rows = p.N >= 4 * 2048 ? 4 : (p.N >= 2 * 2048 || p.M > 2) ? 2 : 1;
  const dim3 grid((p.N + 4 * rows - 1) / (4 * rows)), block(256);
#define FL_SKINNY(MT_)                                                                              \
  do {                                                                                              \
    if (rows == 4) FL_LAUNCH((SkinnyGemmKernel<MT_, 4>), grid, block, 0, s, C, A, B, p);            \
    else if (rows == 2) FL_LAUNCH((SkinnyGemmKernel<MT_, 2>), grid, block, 0, s, C, A, B, p);       \
    else FL_LAUNCH((SkinnyGemmKernel<MT_, 1>), grid, block, 0, s, C, A, B, p);                      \
  } while (0)
  if (p.M == 1) FL_SKINNY(1);
  else if (p.M == 2) FL_SKINNY(2);
  else if (p.M <= 4) FL_SKINNY(4);
  else FL_SKINNY(8);
#undef FL_SKINNY
  return true;
}

// ---- split-K workspace of the entry point that allocates nothing ------------------------------------------
// fluidml_hip_matmul_no_alloc takes the partial tiles and arrival counters of a split-K launch from this
// file-scope array instead of the stream's workspace (which is allocated on a stream's first use).  Every GPU
// the library runs on holds its own copy of the array, at its own address, until the process ends.  In host
// code the array's NAME is only a stand-in for the symbol, not a device address: the address is looked up once
// per device with hipGetSymbolAddress (StaticScratch below) and only that pointer is handed to kernels.
constexpr size_t kStaticSlots = FL_NO_ALLOC_SCRATCH_BYTES / (kWorkspaceTileFloats * sizeof(float));  // partial tiles
constexpr size_t kStaticCounters = 2048;
static __device__ __align__(256) unsigned char scratch[FL_NO_ALLOC_SCRATCH_BYTES + kStaticCounters * sizeof(uint32_t)];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

// Workspace a caller on this thread wants LaunchConfig to use instead of the stream's (null: the stream's).
struct WorkspaceOverride {
  float *partials;
  uint32_t *counters;
  size_t slots;     // partial tiles `partials` holds
  size_t n_counters;
  int error;        // set by LaunchConfig when the launch needs more than that; nothing is launched then
};
thread_local WorkspaceOverride *t_workspace_override = nullptr;

// The counters a split-K launch on the shared static scratch is about to use must start at zero whatever an
// earlier call left there.  A fill kernel, not hipMemsetAsync: the caller may be recording a graph.
__global__ __launch_bounds__(256) void ZeroWordsKernel(uint32_t *p, uint32_t n) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// What the caller fixed of a launch's configuration (fl_contract_tile, K splits; 0 = this file's rule decides).
struct TileChoice {
  int tile = FL_TILE_RULE;
  int splits = 0;
};
inline TileChoice ChoiceOf(uint32_t contract_flags) {
  TileChoice c;
  c.tile = static_cast<int>((contract_flags >> FL_CONTRACT_TILE_SHIFT) & 0xfu);
  c.splits = static_cast<int>((contract_flags >> FL_CONTRACT_SPLIT_SHIFT) & 0x3fu);
  return c;
}

// Upper bound on the number of K splits per tile (environment FLUIDML_SPLITK; default 4 for the 32x32 tile and
// 16 for the 64x64 tile; 1 = never split).
inline int64_t SplitKLimit(int64_t fallback) {
  const char *v = std::getenv("FLUIDML_SPLITK");  // (read at every call)
  const long n = v != nullptr ? std::strtol(v, nullptr, 10) : 0;
  return n > 0 ? static_cast<int64_t>(n) : fallback;
}

template <int BM, int BN, int BK, int WM, int WN, int KS, int LA, int LB, int VEC, int DEPTH, int CONV, bool BF16,
          bool SPEC = false, int EXTRA = 0, int DIRECT = 0>
int LaunchConfig(const MatmulArgs &p, uint32_t n_batch, float *C, const float *A, const float *B, hipStream_t s,
                 int forced_splits = 0) {
  MatmulArgs q = p;
  q.batch_rank = p.batch.rank;
  q.chain_n = p.chain.n;
  q.tiles_m = (p.M + BM - 1) / BM;
  q.tiles_n = (p.N + BN - 1) / BN;
  uint32_t splits = 1;
  constexpr int TM = BM / (32 * WM), TN = BN / (32 * WN);
  if constexpr (TM * TN == 1 && (WM * WN == 1 || KS == 1 || DIRECT > 0)) {
    // Few tiles and a long K: give each tile to several workgroups.  Measured on MI355X (M = 128..256): with
    // about 100 tiles, 2 splits of 3 chunks of 128 (K = 768) and 4 splits of 4..6 chunks (K = 2048, 3072) win
    // by 8 % to 40 %; from about 400 tiles on, or with shorter runs of K per split, the exchange of the
    // partial tiles costs more than the extra workgroups bring.  One workspace slot per wave and split.
    const int64_t tiles = static_cast<int64_t>(q.tiles_m) * q.tiles_n * n_batch;
    const int64_t n_chunks = (p.K + BK - 1) / BK;
    // At most 40 tiles (pointwise convolutions over 7x7 and 14x14 images: 12 .. 28 tiles, K = 480 .. 1152): every
    // chunk of 128 to a workgroup of its own, up to 16 per tile -- the launch is a chain of round trips to memory and
    // each chunk a workgroup runs after its first two adds one (EfficientNet-B0 +2.3 %; limits of 8 and 32 and bounds
    // of 28 and 56 tiles within 0.3 % of that).
    const bool few = tiles <= 40 && WM * WN == 1;
    const int64_t min_chunks = few ? std::max(1, 128 / BK) : 384 / BK;  // at least 384 values of k per split otherwise
    int64_t want = std::min<int64_t>(n_chunks / min_chunks, static_cast<int64_t>(kWorkspaceTiles) / (tiles * WM * WN));
    // (64x64 tile, 3x3 convolutions on 14x14 and 28x28 images at batch 1, K = 4608: 8 -> 12 splits 36 -> 33.5 us and
    // 66 -> 61 us)
    want = std::min<int64_t>(want, SplitKLimit(few ? 16 : WM * WN == 1 ? 4 : 16));
    if (tiles > 256) want = 1;
    if (forced_splits > 0) {
      // the caller's number or nothing: a tuner must not time one configuration under two names
      if (forced_splits > n_chunks ||
          (forced_splits > 1 && static_cast<int64_t>(forced_splits) * tiles * WM * WN > static_cast<int64_t>(kWorkspaceTiles)) ||
          (n_chunks + forced_splits - 1) / forced_splits * (forced_splits - 1) >= n_chunks) {
        return FL_ERR_UNSUPPORTED;
      }
      want = forced_splits;
    }
    if (want >= 2) {
      if (WorkspaceOverride *fixed = t_workspace_override) {
        // same split as with the stream's workspace, so the result is the same bit for bit; refused when
        // the fixed workspace cannot hold it
        q.chunks_per_split = static_cast<int32_t>((n_chunks + want - 1) / want);
        splits = static_cast<uint32_t>((n_chunks + q.chunks_per_split - 1) / q.chunks_per_split);
        const size_t waves = static_cast<size_t>(tiles) * WM * WN;  // one slot per wave and split
        if (waves * splits > fixed->slots || waves * 4 > fixed->n_counters) {
          fixed->error = FL_ERR_STATIC_SCRATCH;
          return FL_ERR_STATIC_SCRATCH;
        }
        q.partials = fixed->partials;
        q.counters = fixed->counters;
        const uint32_t n_zero = static_cast<uint32_t>(waves * 4);  // a wave owns up to four quarter counters
        FL_LAUNCH(ZeroWordsKernel, dim3((n_zero + 255) / 256), dim3(256), 0, s, fixed->counters, n_zero);
      } else if (StreamWorkspace *ws = GetStreamWorkspace(s)) {
        q.chunks_per_split = static_cast<int32_t>((n_chunks + want - 1) / want);
        splits = static_cast<uint32_t>((n_chunks + q.chunks_per_split - 1) / q.chunks_per_split);
        q.partials = ws->partials;
        q.counters = ws->counters;
      } else if (forced_splits > 1) {
        return FL_ERR_UNSUPPORTED;  // no workspace (the stream is being captured before its first use)
      }
    }
  } else if (forced_splits > 1) {
    return FL_ERR_UNSUPPORTED;
  }
  q.n_splits = splits;
  FL_LAUNCH((MatmulKernel<BM, BN, BK, WM, WN, KS, LA, LB, VEC, DEPTH, CONV, BF16, SPEC, EXTRA, DIRECT>),
            dim3(q.tiles_m * q.tiles_n, n_batch, splits), dim3(64 * WM * WN * KS * (SPEC ? 2 : 1)), 0, s, C, A, B, q);
  return FL_OK;
}

// Picks the tile configuration (the caller's, or by the rule below) and launches it.  FL_ERR_UNSUPPORTED, with
// nothing launched, when the caller's choice does not exist for these operands.
template <int LA, int LB, int VEC, int CONV, bool BF16 = false, int EXTRA = 0>
int LaunchBySize(const MatmulArgs &p, uint32_t n_batch, float *C, const float *A, const float *B, hipStream_t s,
                 TileChoice choice = TileChoice()) {
  // the direct-to-LDS loop: both operands on their 128-bit path, plain fp32 contraction
  constexpr bool kDirect = LA == 0 && LB == 0 && VEC == 4 && CONV == 0 && !BF16 && EXTRA != 2;
  int tile = choice.tile;
  if (tile == FL_TILE_RULE) {
    const int64_t tiles_m = static_cast<int64_t>((p.M + 63) / 64) * ((p.N + 63) / 64) * n_batch;
    // (A 128x128x16 tile with two chunks in flight was measured slower than the 64x64x32 tile with four at
    // every size tried -- 4096^3: 101 against 123 TFLOP/s, [256,512]x[512,50304]: 69 against 108, 3x3
    // convolutions: 50 against 67..85 -- and is not built.)
    if (tiles_m >= 192 ||
        (CONV && tiles_m * std::min<int64_t>({8, p.K / 384, static_cast<int64_t>(kWorkspaceTiles) / (tiles_m * 4)}) >= 192)) {
      // also when splitting K over up to 8 workgroups per tile fills the chip (measured on 3x3 convolutions
      // with 32..104 tiles: 1.5x to 2x over the 32x32 tile).  The direct loop on the same tile is level with it
      // ([256,512]x[512,50304]: 133.3 against 133.0 us; 2048^3: 153.7 against 155.2; 4096^3: 1173 against 1130).
      tile = FL_TILE_64x64_STAGED;
    } else {
      // the 32x32 tile whose four waves split K: direct loop where the operands allow it (BERT-base's four shapes:
      // 7.9 -> 7.45, 13.1 -> 12.0, 13.55 -> 12.3, 14.7 -> 13.4 us), else staged through registers by producer waves
      tile = kDirect && p.K % 128 == 0 ? FL_TILE_32x32_K4 : FL_TILE_32x32_STAGED;
    }
  }
  if constexpr (BF16) {
    // bf16 needs a quarter of the matrix-pipe time per tile, so what bounds it is the delivery of the fp32 operands:
    // where there are enough of them, 128x128 tiles (2x2 waves with 2x2 accumulators each) halve that traffic, and four
    // chunks on their way in registers keep it coming (two: 4096^3 310 TFLOP/s, four: 445; [256,512]x[512,50304] 89 -> 57 us)
    const int64_t big_tiles = static_cast<int64_t>((p.M + 127) / 128) * ((p.N + 127) / 128) * n_batch;
    // (two lanes merge the statistics of one of its 128 rows: deferred LayerNormalizations up to 512 wide)
    const bool rows_fit = EXTRA != 1 || p.ln_mode == 0 || p.ln_width <= 512;
    if (choice.tile == FL_TILE_RULE && big_tiles >= 256 && rows_fit) tile = FL_TILE_128x128_STAGED;
    if (tile == FL_TILE_128x128_STAGED) {
      if (choice.splits > 1 || !rows_fit) return FL_ERR_UNSUPPORTED;
      return LaunchConfig<128, 128, 32, 2, 2, 1, LA, LB, VEC, 4, CONV, true, false, EXTRA>(p, n_batch, C, A, B, s, 0);
    }
  }
  switch (tile) {
    case FL_TILE_32x32_STAGED:
      // plain contractions run producer and consumer waves (measured on BERT-base: 8.9 -> 8.6, 14.5 -> 13.6 and
      // 15.9 -> 15.0 us for its three shapes); the convolution gather stays in the consumer waves
      return LaunchConfig<32, 32, 128, 1, 1, 4, LA, LB, VEC, 2, CONV, BF16, CONV == 0, EXTRA>(p, n_batch, C, A, B, s,
                                                                                              choice.splits);
    case FL_TILE_64x64_STAGED:
      return LaunchConfig<64, 64, 32, 2, 2, 1, LA, LB, VEC, 4, CONV, BF16, false, EXTRA>(p, n_batch, C, A, B, s, choice.splits);
    default: break;
  }
  if constexpr (kDirect) {
#define FL_DIRECT(TILE_, WM_, WN_, KS_, R_)                                                                          \
  if (tile == TILE_) {                                                                                               \
    if (p.K % (32 * KS_) != 0) return FL_ERR_UNSUPPORTED;                                                            \
    return LaunchConfig<32 * WM_, 32 * WN_, 32 * KS_, WM_, WN_, KS_, 0, 0, 4, 2, 0, false, false, EXTRA, R_>(        \
        p, n_batch, C, A, B, s, choice.splits);                                                                      \
  }
    // ring depths: the shallowest ones measured best everywhere (more workgroups fit a compute unit)
    FL_DIRECT(FL_TILE_32x32_K4, 1, 1, 4, 2)
    FL_DIRECT(FL_TILE_64x32_K2, 2, 1, 2, 2)
    FL_DIRECT(FL_TILE_64x64, 2, 2, 1, 2)
    FL_DIRECT(FL_TILE_64x64_K2, 2, 2, 2, 2)
    FL_DIRECT(FL_TILE_128x64, 4, 2, 1, 3)
#undef FL_DIRECT
  }
  return FL_ERR_UNSUPPORTED;
}

// Siblings of a grouped launch: same lhs, same extents and rhs strides, own rhs / bias / out buffers.
struct Siblings {
  int count = 0;  // members beyond the first, at most 3
  const fl_tensor *rhs[3];
  const fl_tensor *bias[3];
  const fl_tensor *out[3];
  int64_t stride_outer[3];
};

int Contract(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, bool trans_a, bool trans_b, float ca,
             float cb, const fl_tensor *bias, void *stream, const fl_ew_program *chain = nullptr, int64_t n_inner = 0,
             int64_t stride_outer = 0, const Siblings *siblings = nullptr, bool bf16 = false,
             const float *addend = nullptr, const float *k_scale = nullptr, int64_t k_scale_stride = 0,
             const float *addend2 = nullptr, TileChoice choice = TileChoice(), const fl_norm_fusion *norm = nullptr,
             const fl_tensor *const *col_sum = nullptr, bool addend_is_factor = false) {
  FL_CHECK(CheckChain(chain));
  FL_CHECK(CheckView(lhs));
  FL_CHECK(CheckView(rhs));
  FL_CHECK(CheckView(out));
  if (lhs->dtype != FL_FLOAT32 || rhs->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  if (lhs->rank < 2 || rhs->rank < 2 || out->rank < 2) return FL_ERR_RANK;
  if (lhs->rank > out->rank || rhs->rank > out->rank) return FL_ERR_RANK;
  const int lr = lhs->rank, rr = rhs->rank, orank = out->rank;
  MatmulArgs p;
  std::memset(&p, 0, sizeof(p));
  const int am = trans_a ? lr - 1 : lr - 2, ak = trans_a ? lr - 2 : lr - 1;
  const int bk = trans_b ? rr - 1 : rr - 2, bn = trans_b ? rr - 2 : rr - 1;
  p.M = static_cast<int32_t>(out->shape[orank - 2]);
  p.N = static_cast<int32_t>(out->shape[orank - 1]);
  p.K = static_cast<int32_t>(lhs->shape[ak]);
  if (lhs->shape[am] != p.M || rhs->shape[bn] != p.N || rhs->shape[bk] != p.K) return FL_ERR_SHAPE;
  p.sAm = static_cast<int32_t>(lhs->strides[am]);
  p.sAk = static_cast<int32_t>(lhs->strides[ak]);
  p.sBk = static_cast<int32_t>(rhs->strides[bk]);
  p.sBn = static_cast<int32_t>(rhs->strides[bn]);
  p.sCm = static_cast<int32_t>(out->strides[orank - 2]);
  p.sCn = static_cast<int32_t>(out->strides[orank - 1]);
  // batch dims: trailing alignment, size 1 -> stride 0, missing -> stride 0
  LoopNest nest;
  nest.n_operands = 3;
  nest.rank = orank - 2;
  for (int i = 0; i < orank - 2; ++i) {
    nest.shape[i] = out->shape[i];
    nest.strides[0][i] = out->strides[i];
    const int li = lr - orank + i, ri = rr - orank + i;
    if (li < 0) {
      nest.strides[1][i] = 0;
    } else if (lhs->shape[li] == out->shape[i]) {
      nest.strides[1][i] = lhs->strides[li];
    } else if (lhs->shape[li] == 1) {
      nest.strides[1][i] = 0;
    } else {
      return FL_ERR_SHAPE;
    }
    if (ri < 0) {
      nest.strides[2][i] = 0;
    } else if (rhs->shape[ri] == out->shape[i]) {
      nest.strides[2][i] = rhs->strides[ri];
    } else if (rhs->shape[ri] == 1) {
      nest.strides[2][i] = 0;
    } else {
      return FL_ERR_SHAPE;
    }
  }
  nest.Canonicalise();
  int64_t n_batch = 1;
  for (int i = 0; i < nest.rank; ++i) n_batch *= nest.shape[i];
  if (n_batch > 65535) return FL_ERR_TOO_LARGE;
  FL_CHECK(MakeBatchArgs(nest, n_batch, &p.batch));
  p.ca = ca;
  p.cb = cb;
  if (chain != nullptr) p.chain = *chain;
  if (n_inner != 0) {
    if (n_inner < 0 || p.N % n_inner != 0 || stride_outer < 0 || stride_outer > INT32_MAX) return FL_ERR_ATTR;
    p.n_inner = static_cast<int32_t>(n_inner);
    p.sCn_outer = static_cast<int32_t>(stride_outer);
    p.div_inner = FastDiv(static_cast<uint32_t>(n_inner));
  }
  if (bias != nullptr) {
    FL_CHECK(CheckView(bias));
    if (bias->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    if (bias->rank == 1) {
      if (bias->shape[0] != p.N) return FL_ERR_SHAPE;
      p.sDm = 0;
      p.sDn = static_cast<int32_t>(bias->strides[0]);
    } else if (bias->rank == 2) {
      if (bias->shape[0] != p.M || bias->shape[1] != p.N) return FL_ERR_SHAPE;
      p.sDm = static_cast<int32_t>(bias->strides[0]);
      p.sDn = static_cast<int32_t>(bias->strides[1]);
    } else {
      return FL_ERR_RANK;
    }
    p.bias = static_cast<const float *>(bias->base);
  }

  float *C = static_cast<float *>(out->base);
  const float *A = static_cast<const float *>(lhs->base);
  const float *B = static_cast<const float *>(rhs->base);
  hipStream_t s = AsStream(stream);

  bool siblings_aligned = true;
  if (siblings != nullptr && siblings->count > 0) {
    if (siblings->count > 3 || n_batch != 1) return FL_ERR_UNSUPPORTED;
    for (int g = 0; g < siblings->count; ++g) {
      const fl_tensor *r = siblings->rhs[g], *o = siblings->out[g], *bs = siblings->bias[g];
      FL_CHECK(CheckView(r));
      FL_CHECK(CheckView(o));
      if (r->dtype != FL_FLOAT32 || o->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
      if (r->rank != rhs->rank || o->rank != out->rank || (bs == nullptr) != (bias == nullptr)) return FL_ERR_SHAPE;
      for (int i = 0; i < rr; ++i) {
        if (r->shape[i] != rhs->shape[i] || r->strides[i] != rhs->strides[i]) return FL_ERR_SHAPE;
      }
      for (int i = 0; i < orank; ++i) {
        if (o->shape[i] != out->shape[i]) return FL_ERR_SHAPE;
      }
      if (bs != nullptr) {
        FL_CHECK(CheckView(bs));
        if (bs->dtype != FL_FLOAT32 || bs->rank != bias->rank || bs->shape[0] != bias->shape[0] ||
            bs->strides[0] != bias->strides[0]) return FL_ERR_SHAPE;
        p.gbias[g] = static_cast<const float *>(bs->base);
      }
      p.gB[g] = static_cast<const float *>(r->base);
      p.gC[g] = static_cast<float *>(o->base);
      p.g_sCm[g] = static_cast<int32_t>(o->strides[orank - 2]);
      p.g_sCn[g] = static_cast<int32_t>(o->strides[orank - 1]);
      p.g_sCn_outer[g] = static_cast<int32_t>(siblings->stride_outer[g]);
      siblings_aligned = siblings_aligned && IsAligned(r->base, 16);
    }
    p.n_groups = siblings->count + 1;
    n_batch = p.n_groups;  // one grid row per sibling
  }

  // Layout of each staged tile follows the operand's fast dimension; 128-bit
  // loads need that dimension to have unit stride and everything else to keep
  // 16-byte alignment.
  const int la = (p.sAk <= p.sAm || p.M == 1) ? 0 : 1;
  const int lb = (p.sBn <= p.sBk || p.K == 1) ? 0 : 1;
  bool vec_a = IsAligned(A, 16), vec_b = IsAligned(B, 16) && siblings_aligned;
  if (la == 0) vec_a = vec_a && (p.sAk == 1 || p.K == 1) && p.K % 4 == 0 && p.sAm % 4 == 0;
  else vec_a = vec_a && p.sAm == 1 && p.M % 4 == 0 && p.sAk % 4 == 0;
  if (lb == 0) vec_b = vec_b && (p.sBn == 1 || p.N == 1) && p.N % 4 == 0 && p.sBk % 4 == 0;
  else vec_b = vec_b && p.sBk == 1 && p.K % 4 == 0 && p.sBn % 4 == 0;
  for (int i = 0; i < nest.rank; ++i) {
    if (nest.strides[1][i] % 4 != 0) vec_a = false;
    if (nest.strides[2][i] % 4 != 0) vec_b = false;
  }
  const bool vec = vec_a && vec_b;
  // k-contiguous weights over an operand whose rows lose the alignment (49 pixels): wide loads for the weights alone
  const bool vec_a_only = vec_a && !vec_b && la == 0 && lb == 0 && !bf16;
  // a second addend with the strides of C / a scale per row of B: the tiled kernel's own instantiations (fp32)
  const bool extra = addend != nullptr || k_scale != nullptr || norm != nullptr;
  if (extra) {
    // (grouped members and split output columns have their own strides of C: the addends are read through the
    // plain ones)
    if (lb != 0 || (addend2 != nullptr && addend == nullptr)) return FL_ERR_UNSUPPORTED;
    if (addend != nullptr && (p.n_groups > 1 || p.n_inner != 0)) return FL_ERR_UNSUPPORTED;
    if (addend_is_factor && (addend == nullptr || addend2 != nullptr || norm != nullptr)) return FL_ERR_UNSUPPORTED;
    p.addend = addend;
    p.addend2 = addend2;
    p.addend_is_factor = addend_is_factor ? 1 : 0;
  } else if (addend_is_factor) {
    return FL_ERR_UNSUPPORTED;
  }
  if (norm != nullptr) {
    // a LayerNormalization folded into this launch: one batch element, rows short enough for the lanes that
    // merge a row's partial statistics (64x64 tile: 4 lanes x 8 partials x 32 columns)
    const int64_t real_batch = siblings != nullptr && siblings->count > 0 ? 1 : n_batch;
    if (real_batch != 1 || k_scale != nullptr) return FL_ERR_UNSUPPORTED;
    if (norm->deferred != FL_NORM_NONE) {
      if (norm->stats == nullptr || norm->width <= 0 || norm->width > 1024) return FL_ERR_UNSUPPORTED;
      p.ln_mode = norm->deferred;
      p.ln_width = norm->width;
      p.ln_parts = (norm->width + 31) / 32;
      p.ln_eps = static_cast<float>(norm->epsilon);
      p.ln_inv_width = 1.0f / static_cast<float>(norm->width);
      p.ln_stats = norm->stats;
    }
    auto vector_of = [&](const fl_tensor *t, int64_t extent, const float **base, int32_t *stride) -> int {
      if (t == nullptr) return FL_ERR_NULL;
      FL_CHECK(CheckView(t));
      if (t->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
      if (t->rank != 1 || t->shape[0] != extent) return FL_ERR_SHAPE;
      *base = static_cast<const float *>(t->base);
      *stride = static_cast<int32_t>(t->strides[0]);
      return FL_OK;
    };
    if (norm->deferred == FL_NORM_LHS) {
      // the row statistics belong to A's rows: the normalised axis is K; c1 per member, the bias carries shift . B
      if (norm->width != p.K || col_sum == nullptr || bias == nullptr || p.sDm != 0 || addend != nullptr) return FL_ERR_UNSUPPORTED;
      if (p.ca != 1.0f || p.cb != 1.0f) return FL_ERR_UNSUPPORTED;
      FL_CHECK(vector_of(col_sum[0], p.N, &p.ln_c1, &p.ln_s_c1));
      for (int g = 1; g < p.n_groups; ++g) {
        int32_t stride = 0;
        FL_CHECK(vector_of(col_sum[g], p.N, &p.g_ln_c1[g - 1], &stride));
        if (stride != p.ln_s_c1) return FL_ERR_SHAPE;
      }
    } else if (norm->deferred == FL_NORM_ADDEND) {
      // the addend has C's shape: the normalised axis is N
      if (norm->width != p.N || addend == nullptr) return FL_ERR_UNSUPPORTED;
      FL_CHECK(vector_of(norm->scale, p.N, &p.ln_scale, &p.ln_s_scale));
      FL_CHECK(vector_of(norm->shift, p.N, &p.ln_shift, &p.ln_s_shift));
    } else if (norm->deferred != FL_NORM_NONE) {
      return FL_ERR_ATTR;
    }
    if (norm->stats_out != nullptr && (p.n_groups > 1 || p.n_inner != 0)) return FL_ERR_UNSUPPORTED;
    p.ln_stats_out = norm->stats_out;
  }
  if (k_scale != nullptr) {
    if (n_batch != 1 || k_scale_stride > INT32_MAX || k_scale_stride < 0) return FL_ERR_UNSUPPORTED;
    p.k_scale = k_scale;
    p.sKs = static_cast<int32_t>(k_scale_stride);
  }
  // at most 8 rows against k-contiguous weights: HBM-bound weight streaming, fp32 whatever `bf16` says (a caller
  // that names a tile configuration gets the tiled kernel)
  const bool free_choice = choice.tile == FL_TILE_RULE && choice.splits == 0;
  if (!extra && free_choice && TrySkinnyGemm(p, n_batch, C, A, B, s)) return LaunchStatus();
  const uint32_t nb = static_cast<uint32_t>(n_batch);
  int rc = FL_ERR_UNSUPPORTED;
  if (extra) {
#define FL_MM_EXTRA(E_)                                                                 \
  do {                                                                                  \
    if (la == 0 && vec) rc = LaunchBySize<0, 0, 4, 0, false, E_>(p, nb, C, A, B, s, choice);   \
    else if (vec_a_only) rc = LaunchBySize<0, 0, 41, 0, false, E_>(p, nb, C, A, B, s, choice); \
    else if (la == 0) rc = LaunchBySize<0, 0, 1, 0, false, E_>(p, nb, C, A, B, s, choice);     \
    else if (vec) rc = LaunchBySize<1, 0, 4, 0, false, E_>(p, nb, C, A, B, s, choice);         \
    else rc = LaunchBySize<1, 0, 1, 0, false, E_>(p, nb, C, A, B, s, choice);                  \
  } while (0)
    // (bf16 operands with the epilogue operands: the common case of dense row-major operands only)
    if (k_scale != nullptr) FL_MM_EXTRA(2);
    else if (bf16 && la == 0 && vec) rc = LaunchBySize<0, 0, 4, 0, true, 1>(p, nb, C, A, B, s, choice);
    else FL_MM_EXTRA(1);
#undef FL_MM_EXTRA
    return rc != FL_OK ? rc : LaunchStatus();
  }
#define FL_MM_DISPATCH(LA_, LB_)                                                  \
  if (la == LA_ && lb == LB_) {                                                   \
    if (bf16) {                                                                   \
      if (vec) rc = LaunchBySize<LA_, LB_, 4, 0, true>(p, nb, C, A, B, s, choice); \
      else rc = LaunchBySize<LA_, LB_, 1, 0, true>(p, nb, C, A, B, s, choice);     \
    } else if (vec) {                                                             \
      rc = LaunchBySize<LA_, LB_, 4, 0>(p, nb, C, A, B, s, choice);               \
    } else {                                                                      \
      rc = LaunchBySize<LA_, LB_, 1, 0>(p, nb, C, A, B, s, choice);               \
    }                                                                             \
  }
  if (vec_a_only) {
    rc = LaunchBySize<0, 0, 41, 0>(p, nb, C, A, B, s, choice);
    return rc != FL_OK ? rc : LaunchStatus();
  }
  FL_MM_DISPATCH(0, 0)
  FL_MM_DISPATCH(0, 1)
  FL_MM_DISPATCH(1, 0)
  FL_MM_DISPATCH(1, 1)
#undef FL_MM_DISPATCH
  return rc != FL_OK ? rc : LaunchStatus();
}

}  // namespace

// Convolution with group == 1 and one or two spatial dims as an implicit GEMM on the matrix cores.
// Returns FL_ERR_UNSUPPORTED (nothing launched) when the operands do not fit this path: the caller then
// uses the direct kernel.  `pads` may be null; `strides`/`dilations` have one entry per spatial dim.
int ConvImplicitGemm(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out,
                     const int64_t *pads, const int64_t *strides, const int64_t *dilations,
                     const fl_ew_program *chain, bool bf16, void *stream, const ConvExtras *extras) {
  const int ns = out->rank - 2;
  if (ns != 1 && ns != 2) return FL_ERR_UNSUPPORTED;
  const float *addend = nullptr;
  if (extras != nullptr && extras->addend != nullptr) {
    const fl_tensor *e = extras->addend;
    FL_CHECK(CheckView(e));
    if (e->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    if (e->rank != out->rank) return FL_ERR_SHAPE;
    for (int i = 0; i < out->rank; ++i) {
      if (e->shape[i] != out->shape[i]) return FL_ERR_SHAPE;
      if (out->shape[i] > 1 && e->strides[i] != out->strides[i]) return FL_ERR_UNSUPPORTED;
    }
    addend = static_cast<const float *>(e->base);
  }
  const fl_tensor *scale = extras != nullptr ? extras->channel_scale : nullptr;
  if (scale != nullptr) {
    FL_CHECK(CheckView(scale));
    if (scale->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    if (scale->rank != in->rank || scale->shape[1] != in->shape[1]) return FL_ERR_SHAPE;
    for (int i = 0; i < scale->rank; ++i) {
      if (i != 1 && scale->shape[i] != 1) return FL_ERR_SHAPE;
    }
    if (in->shape[0] != 1) return FL_ERR_UNSUPPORTED;  // one scale vector per image: one image per launch
  }
  const int hd = ns == 2 ? 2 : -1, wd = ns == 2 ? 3 : 2;  // dims of H (absent for 1-d) and W
  const int64_t KH = ns == 2 ? weights->shape[2] : 1, KW = weights->shape[wd];
  const int64_t Cc = in->shape[1], F = out->shape[1];
  const int64_t OH = ns == 2 ? out->shape[2] : 1, OW = out->shape[wd];
  const int64_t n_total = out->shape[0] * OH * OW, k_total = Cc * KH * KW;
  if (n_total > 0x7fffffff || k_total > 0x7fffffff || n_total == 0 || F == 0) return FL_ERR_UNSUPPORTED;
  // A = weights as an [F][K] matrix: (c, kh, kw) must be one strided run
  const int64_t s_kw = weights->strides[wd];
  if (ns == 2 && KH > 1 && weights->strides[2] != KW * s_kw) return FL_ERR_UNSUPPORTED;
  if (Cc > 1 && weights->strides[1] != KH * KW * s_kw) return FL_ERR_UNSUPPORTED;
  if (Numel(in) > 0x7fffffff || Numel(out) > 0x7fffffff) return FL_ERR_UNSUPPORTED;

  // A 1x1 convolution with unit stride and no padding is a plain batched contraction
  // out[img] = W[F][C] . in[img][C][H*W]: no gather, 128-bit loads of both operands, the producer/consumer tile.
  {
    bool pointwise = KH == 1 && KW == 1;
    for (int d = 0; d < ns && pointwise; ++d) {
      pointwise = (!strides || strides[d] == 1) && (!pads || (pads[d] == 0 && pads[ns + d] == 0));
    }
    if (pointwise && ns == 2) {
      pointwise = in->strides[2] == in->shape[3] * in->strides[3] && out->strides[2] == out->shape[3] * out->strides[3];
    }
    if (pointwise) {
      const int64_t S = OH * OW;
      fl_tensor a{}, b{}, c{}, d{};
      a.base = weights->base, a.dtype = FL_FLOAT32, a.rank = 2;
      a.shape[0] = F, a.shape[1] = Cc, a.strides[0] = weights->strides[0], a.strides[1] = weights->strides[1];
      b.base = in->base, b.dtype = FL_FLOAT32, b.rank = 3;
      b.shape[0] = in->shape[0], b.shape[1] = Cc, b.shape[2] = S;
      b.strides[0] = in->strides[0], b.strides[1] = in->strides[1], b.strides[2] = in->strides[wd];
      c.base = out->base, c.dtype = FL_FLOAT32, c.rank = 3;
      c.shape[0] = out->shape[0], c.shape[1] = F, c.shape[2] = S;
      c.strides[0] = out->strides[0], c.strides[1] = out->strides[1], c.strides[2] = out->strides[wd];
      if (bias != nullptr) {
        d.base = bias->base, d.dtype = FL_FLOAT32, d.rank = 2;
        d.shape[0] = F, d.shape[1] = S, d.strides[0] = bias->strides[0], d.strides[1] = 0;
      }
      return Contract(&a, &b, &c, false, false, 1.0f, 1.0f, bias != nullptr ? &d : nullptr, stream, chain, 0, 0, nullptr,
                      bf16, addend, scale != nullptr ? static_cast<const float *>(scale->base) : nullptr,
                      scale != nullptr ? scale->strides[1] : 0, nullptr, TileChoice(), nullptr, nullptr,
                      extras != nullptr && extras->addend_is_factor);
    }
  }
  if (scale != nullptr || addend != nullptr) return FL_ERR_UNSUPPORTED;  // only the pointwise form carries them

  MatmulArgs p;
  std::memset(&p, 0, sizeof(p));
  p.M = static_cast<int32_t>(F);
  p.N = static_cast<int32_t>(n_total);
  p.K = static_cast<int32_t>(k_total);
  p.sAm = static_cast<int32_t>(weights->strides[0]);
  p.sAk = static_cast<int32_t>(s_kw);
  p.sCm = static_cast<int32_t>(out->strides[1]);
  p.sCn = 0;
  p.batch.rank = 0;
  p.ca = 1.0f;
  p.cb = 1.0f;
  if (chain != nullptr) p.chain = *chain;
  if (bias != nullptr) {
    p.bias = static_cast<const float *>(bias->base);
    p.sDm = static_cast<int32_t>(bias->strides[0]);
    p.sDn = 0;
  }
  ConvGeom &g = p.conv;
  g.H = ns == 2 ? static_cast<int32_t>(in->shape[2]) : 1;
  g.W = static_cast<int32_t>(in->shape[wd]);
  g.sh = ns == 2 && strides ? static_cast<int32_t>(strides[0]) : 1;
  g.sw = strides ? static_cast<int32_t>(strides[ns - 1]) : 1;
  g.dh = ns == 2 && dilations ? static_cast<int32_t>(dilations[0]) : 1;
  g.dw = dilations ? static_cast<int32_t>(dilations[ns - 1]) : 1;
  g.ph = ns == 2 && pads ? static_cast<int32_t>(pads[0]) : 0;
  g.pw = pads ? static_cast<int32_t>(pads[ns - 1]) : 0;
  g.sXn = static_cast<int32_t>(in->strides[0]);
  g.sXc = static_cast<int32_t>(in->strides[1]);
  g.sXh = ns == 2 ? static_cast<int32_t>(in->strides[2]) : 0;
  g.sXw = static_cast<int32_t>(in->strides[wd]);
  g.sOn = static_cast<int32_t>(out->strides[0]);
  g.sOh = ns == 2 ? static_cast<int32_t>(out->strides[2]) : 0;
  g.sOw = static_cast<int32_t>(out->strides[wd]);
  g.div_ohw = FastDiv(static_cast<uint32_t>(OH * OW));
  g.div_ow = FastDiv(static_cast<uint32_t>(OW));
  g.div_khw = FastDiv(static_cast<uint32_t>(KH * KW));
  g.div_kw = FastDiv(static_cast<uint32_t>(KW));
  (void)hd;

  float *C = static_cast<float *>(out->base);
  const float *A = static_cast<const float *>(weights->base);
  const float *B = static_cast<const float *>(in->base);
  hipStream_t s = AsStream(stream);
  const int la = (p.sAk <= p.sAm || p.M == 1) ? 0 : 1;
  bool vec = IsAligned(A, 16);
  if (la == 0) vec = vec && (p.sAk == 1 || p.K == 1) && p.K % 4 == 0 && p.sAm % 4 == 0;
  else vec = vec && p.sAm == 1 && p.M % 4 == 0 && p.sAk % 4 == 0;
  // four output pixels per gather when they sit in one input row at unit stride
  const bool quad = g.sw == 1 && g.sXw == 1 && OW % 4 == 0;
  int rc = FL_ERR_UNSUPPORTED;
#define FL_CONV_DISPATCH(LA_, VEC_)                                         \
  do {                                                                      \
    if (bf16) {                                                             \
      if (quad) rc = LaunchBySize<LA_, 0, VEC_, 2, true>(p, 1, C, A, B, s); \
      else rc = LaunchBySize<LA_, 0, VEC_, 1, true>(p, 1, C, A, B, s);      \
    } else if (quad) {                                                      \
      rc = LaunchBySize<LA_, 0, VEC_, 2>(p, 1, C, A, B, s);                 \
    } else {                                                                \
      rc = LaunchBySize<LA_, 0, VEC_, 1>(p, 1, C, A, B, s);                 \
    }                                                                       \
  } while (0)
  if (la == 0) {
    if (vec) FL_CONV_DISPATCH(0, 4);
    else FL_CONV_DISPATCH(0, 1);
  } else {
    if (vec) FL_CONV_DISPATCH(1, 4);
    else FL_CONV_DISPATCH(1, 1);
  }
#undef FL_CONV_DISPATCH
  return rc != FL_OK ? rc : LaunchStatus();
}

// Device address of the current device's copy of `scratch`, looked up on the first call per device.
int StaticScratch(void **ptr) {
  int dev = -1;
  FL_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return FL_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void *p = nullptr;
    FL_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (p == nullptr) return FL_ERR_NULL;
    g_scratch_ptr[dev] = p;
  }
  if (ptr != nullptr) *ptr = g_scratch_ptr[dev];
  return FL_OK;
}

}  // namespace fl

extern "C" {

int fluidml_hip_matmul(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream) {
  return fl::Contract(lhs, rhs, out, false, false, 1.0f, 0.0f, nullptr, stream);
}

int fluidml_hip_matmul_no_alloc(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream) {
  if (!lhs || !rhs || !out) return FL_ERR_NULL;
  void *base = nullptr;
  FL_CHECK(fl::StaticScratch(&base));
  fl::WorkspaceOverride fixed;
  fixed.partials = static_cast<float *>(base);
  fixed.counters = reinterpret_cast<uint32_t *>(static_cast<unsigned char *>(base) + FL_NO_ALLOC_SCRATCH_BYTES);
  fixed.slots = fl::kStaticSlots;
  fixed.n_counters = fl::kStaticCounters;
  fixed.error = FL_OK;
  fl::t_workspace_override = &fixed;
  const int rc = fl::Contract(lhs, rhs, out, false, false, 1.0f, 0.0f, nullptr, stream);
  fl::t_workspace_override = nullptr;
  return fixed.error != FL_OK ? fixed.error : rc;
}

int fluidml_hip_matmul_add(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out,
                           void *stream) {
  if (!lhs || !rhs || !bias || !out) return FL_ERR_NULL;
  if (bias->rank != 1) return FL_ERR_RANK;
  return fl::Contract(lhs, rhs, out, false, false, 1.0f, 1.0f, bias, stream);
}

int fluidml_hip_matmul_chain(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out,
                             const fl_ew_program *chain, uint32_t flags, void *stream) {
  if (!lhs || !rhs || !out) return FL_ERR_NULL;
  if (bias != nullptr && bias->rank != 1) return FL_ERR_RANK;
  return fl::Contract(lhs, rhs, out, false, false, 1.0f, 1.0f, bias, stream, chain, 0, 0, nullptr,
                      (flags & FL_CONTRACT_BF16) != 0, nullptr, nullptr, 0, nullptr, fl::ChoiceOf(flags));
}

int fluidml_hip_matmul_chain_add(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out,
                                 const fl_ew_program *chain, const fl_tensor *addend, const fl_tensor *addend2,
                                 uint32_t flags, void *stream) {
  if (!lhs || !rhs || !out || !addend) return FL_ERR_NULL;
  if (bias != nullptr && bias->rank != 1) return FL_ERR_RANK;
  const float *e[2] = {nullptr, nullptr};
  const fl_tensor *t[2] = {addend, addend2};
  for (int i = 0; i < 2; ++i) {
    if (t[i] == nullptr) continue;
    FL_CHECK(fl::CheckView(t[i]));
    if (t[i]->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    if (t[i]->rank != out->rank) return FL_ERR_SHAPE;
    for (int d = 0; d < out->rank; ++d) {
      if (t[i]->shape[d] != out->shape[d]) return FL_ERR_SHAPE;
      if (out->shape[d] > 1 && t[i]->strides[d] != out->strides[d]) return FL_ERR_UNSUPPORTED;
    }
    e[i] = static_cast<const float *>(t[i]->base);
  }
  // fp32 whatever the flags say: the extra operands exist in the fp32 instantiations only
  return fl::Contract(lhs, rhs, out, false, false, 1.0f, 1.0f, bias, stream, chain, 0, 0, nullptr,
                      (flags & FL_CONTRACT_BF16) != 0, e[0], nullptr, 0, e[1], fl::ChoiceOf(flags));
}

int fluidml_hip_matmul_chain_view(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out,
                                  int64_t n_inner, int64_t stride_outer, const fl_ew_program *chain, uint32_t flags,
                                  void *stream) {
  if (!lhs || !rhs || !out) return FL_ERR_NULL;
  if (bias != nullptr && bias->rank != 1) return FL_ERR_RANK;
  return fl::Contract(lhs, rhs, out, false, false, 1.0f, 1.0f, bias, stream, chain, n_inner, stride_outer, nullptr,
                      (flags & FL_CONTRACT_BF16) != 0, nullptr, nullptr, 0, nullptr, fl::ChoiceOf(flags));
}

int fluidml_hip_matmul_chain_group(int32_t count, const fl_tensor *lhs, const fl_tensor *const *rhs,
                                   const fl_tensor *const *bias, const fl_tensor *const *out, int64_t n_inner,
                                   const int64_t *stride_outer, const fl_ew_program *chain, uint32_t flags,
                                   void *stream) {
  if (!lhs || !rhs || !out) return FL_ERR_NULL;
  if (count < 1 || count > 4) return FL_ERR_ATTR;
  fl::Siblings sib;
  sib.count = count - 1;
  for (int g = 0; g < count; ++g) {
    if (!rhs[g] || !out[g]) return FL_ERR_NULL;
    if (bias != nullptr && bias[g] != nullptr && bias[g]->rank != 1) return FL_ERR_RANK;
    if (g > 0) {
      sib.rhs[g - 1] = rhs[g];
      sib.out[g - 1] = out[g];
      sib.bias[g - 1] = bias != nullptr ? bias[g] : nullptr;
      sib.stride_outer[g - 1] = stride_outer != nullptr ? stride_outer[g] : 0;
    }
  }
  return fl::Contract(lhs, rhs[0], out[0], false, false, 1.0f, 1.0f, bias != nullptr ? bias[0] : nullptr, stream, chain,
                      n_inner, stride_outer != nullptr ? stride_outer[0] : 0, &sib, (flags & FL_CONTRACT_BF16) != 0, nullptr,
                      nullptr, 0, nullptr, fl::ChoiceOf(flags));
}

int fluidml_hip_matmul_chain_group_norm(int32_t count, const fl_tensor *lhs, const fl_tensor *const *rhs,
                                        const fl_tensor *const *bias, const fl_tensor *const *col_sum,
                                        const fl_tensor *const *out, int64_t n_inner, const int64_t *stride_outer,
                                        const fl_ew_program *chain, const fl_tensor *addend, const fl_norm_fusion *norm,
                                        uint32_t flags, void *stream) {
  if (!lhs || !rhs || !out || !norm) return FL_ERR_NULL;
  if (count < 1 || count > 4) return FL_ERR_ATTR;
  fl::Siblings sib;
  sib.count = count - 1;
  for (int g = 0; g < count; ++g) {
    if (!rhs[g] || !out[g]) return FL_ERR_NULL;
    if (bias != nullptr && bias[g] != nullptr && bias[g]->rank != 1) return FL_ERR_RANK;
    if (g > 0) {
      sib.rhs[g - 1] = rhs[g];
      sib.out[g - 1] = out[g];
      sib.bias[g - 1] = bias != nullptr ? bias[g] : nullptr;
      sib.stride_outer[g - 1] = stride_outer != nullptr ? stride_outer[g] : 0;
    }
  }
  const float *extra = nullptr;
  if (addend != nullptr) {
    if (count != 1 || n_inner != 0) return FL_ERR_UNSUPPORTED;
    FL_CHECK(fl::CheckView(addend));
    if (addend->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    if (addend->rank != out[0]->rank) return FL_ERR_SHAPE;
    for (int d = 0; d < out[0]->rank; ++d) {
      if (addend->shape[d] != out[0]->shape[d]) return FL_ERR_SHAPE;
      if (out[0]->shape[d] > 1 && addend->strides[d] != out[0]->strides[d]) return FL_ERR_UNSUPPORTED;
    }
    extra = static_cast<const float *>(addend->base);
  }
  const float *extra2 = nullptr;
  if (norm->addend2 != nullptr) {
    const fl_tensor *second = norm->addend2;
    if (addend == nullptr) return FL_ERR_UNSUPPORTED;
    FL_CHECK(fl::CheckView(second));
    if (second->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    if (second->rank != out[0]->rank) return FL_ERR_SHAPE;
    for (int d = 0; d < out[0]->rank; ++d) {
      if (second->shape[d] != out[0]->shape[d]) return FL_ERR_SHAPE;
      if (out[0]->shape[d] > 1 && second->strides[d] != out[0]->strides[d]) return FL_ERR_UNSUPPORTED;
    }
    extra2 = static_cast<const float *>(second->base);
  }
  return fl::Contract(lhs, rhs[0], out[0], false, false, 1.0f, 1.0f, bias != nullptr ? bias[0] : nullptr, stream, chain,
                      n_inner, stride_outer != nullptr ? stride_outer[0] : 0, count > 1 ? &sib : nullptr,
                      (flags & FL_CONTRACT_BF16) != 0, extra, nullptr,
                      0, extra2, fl::ChoiceOf(flags), norm, col_sum);
}

int fluidml_hip_gemm_chain(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out,
                           double alpha, double beta, int32_t trans_a, int32_t trans_b, const fl_ew_program *chain,
                           uint32_t flags, void *stream) {
  if (!lhs || !rhs || !bias || !out) return FL_ERR_NULL;
  if (lhs->rank != 2 || rhs->rank != 2 || out->rank != 2) return FL_ERR_RANK;
  return fl::Contract(lhs, rhs, out, trans_a != 0, trans_b != 0, static_cast<float>(alpha), static_cast<float>(beta),
                      bias, stream, chain, 0, 0, nullptr, (flags & FL_CONTRACT_BF16) != 0, nullptr, nullptr, 0, nullptr,
                      fl::ChoiceOf(flags));
}

int fluidml_hip_matmul_bf16(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream) {
  return fl::Contract(lhs, rhs, out, false, false, 1.0f, 0.0f, nullptr, stream, nullptr, 0, 0, nullptr, true);
}

int fluidml_hip_gemm_constant_weights_bias(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias,
                                           const fl_tensor *out, double alpha, double beta, int32_t trans_a,
                                           int32_t trans_b, uint32_t flags, void *stream) {
  if (!lhs || !rhs || !bias || !out) return FL_ERR_NULL;
  if (lhs->rank != 2 || rhs->rank != 2 || out->rank != 2) return FL_ERR_RANK;  // reference gemm.cpp:57-61
  // acc = A.B; reference: alpha * bias + beta * acc (gemm.cpp:176-179); ONNX: alpha * acc + beta * bias
  const bool swapped = (flags & FL_REF_GEMM_SWAPPED_SCALARS) != 0;
  const float ca = static_cast<float>(swapped ? beta : alpha);
  const float cb = static_cast<float>(swapped ? alpha : beta);
  const bool bf16 = ((flags >> FL_CONTRACT_SHIFT) & FL_CONTRACT_BF16) != 0;
  return fl::Contract(lhs, rhs, out, trans_a != 0, trans_b != 0, ca, cb, bias, stream, nullptr, 0, 0, nullptr, bf16,
                      nullptr, nullptr, 0, nullptr, fl::ChoiceOf(flags >> FL_CONTRACT_SHIFT));
}

}  // extern "C"
