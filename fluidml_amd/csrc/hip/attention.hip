// One launch for the core of an attention block:
//   scores = Q . K^T ; scores = scores / c (or * c) [+ mask] [where(cond, scores, fill)] ;
//   P = softmax(scores, last axis) ; out = P . V
// i.e. the chain MatMulKernel -> DivConstantRhs/MulConstant -> AddCommon / WhereConstantCond -> SoftmaxKernel
// -> MatMulKernel (reference matmul.cpp:28-59, div.cpp:24-56, mul.cpp, add.cpp:75-137, where.cpp:17-150,
// softmax.cpp:22-139) without writing the [.., Sq, Skv] score and probability tensors.
//
// One workgroup (4 waves) owns 16 query rows of one batch element (head), so that even a single sequence
// spreads over many compute units; the kernel is latency bound and every phase is kept short:
//   1. Q block and K^T chunk (128 keys) travel global -> registers -> LDS, 128 bits at a time when the
//      operands allow it; the V chunk, the mask and the condition are requested before the first MFMA.
//   2. wave w computes the 16x32 scores of keys [128c + 32w, +32) with v_mfma_f32_16x16x4_f32 and writes them
//      to an LDS score strip [16][Skv].
//   3. the strip is re-read row-wise (16 lanes per row, contiguous keys per lane): scale, mask, condition,
//      maximum, exp and sum with four shuffle steps each; the unnormalised exp goes back to the strip.
//   4. wave w multiplies the strip with columns [16w, +16) of V (all keys), so no partial sums cross waves,
//      and divides by the row sum while storing.
// Every operand is addressed through element strides, so the head split of the producers and the head merge
// of the consumer need no copies.
#include "fl_common.h"

namespace fl {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kQ = 16;        // query rows per workgroup
constexpr int kKeys = 128;    // keys per chunk (32 per wave)
constexpr int kMaxD = 64;     // head dim limit
constexpr int kLdQ = kMaxD + 4;
constexpr int kLdK = kKeys + 4;
constexpr int kLdV = kMaxD + 4;

struct AttentionArgs {
  NestArgs<6> batch;  // operands: 0 out, 1 q, 2 kt, 3 v, 4 mask, 5 cond
  int32_t Sq, Skv, D;
  int32_t sQm, sQd, sKd, sKn, sVn, sVd, sOm, sOd;
  int32_t sMm, sMn, sCm, sCn;  // additive mask / keep condition strides along (query, key)
  float scale;
  int32_t scale_is_divisor;
  float fill;
  uint32_t q_blocks;
};

// VEC: q, kt and v are unit-stride along (d, key, d), every other stride, the batch offsets, D and Skv are
// multiples of four elements and the bases are 16-byte aligned.
template <int CHUNKS, bool VEC>
__global__ __launch_bounds__(256) void AttentionKernel(AttentionArgs a, float *__restrict__ out, const float *__restrict__ q,
                                                       const float *__restrict__ kt, const float *__restrict__ v,
                                                       const float *__restrict__ mask, const uint8_t *__restrict__ cond) {
  constexpr int kLdP = CHUNKS * kKeys + 4;
  constexpr int kNpt = CHUNKS * kKeys / 16;  // keys per lane in the row-wise phase
  __shared__ __attribute__((aligned(16))) float qs[kQ * kLdQ];
  __shared__ __attribute__((aligned(16))) float kv[kKeys * kLdV > kMaxD * kLdK ? kKeys * kLdV : kMaxD * kLdK];
  __shared__ __attribute__((aligned(16))) float ps[kQ * kLdP];
  __shared__ float row_sum[kQ];

  // Workgroup ids go round the 8 XCDs; renumbered so that each XCD takes a contiguous run of (head, query block)
  // pairs, a head's K and V are fetched by one or two of the L2s instead of all eight.
  uint32_t bid = blockIdx.x;
  if (gridDim.x % 8 == 0) bid = (bid % 8) * (gridDim.x / 8) + bid / 8;
  const uint32_t qb = bid % a.q_blocks;
  int32_t off[6] = {0, 0, 0, 0, 0, 0};
  a.batch.AddOffsets(bid / a.q_blocks, off);
  const int m0 = static_cast<int>(qb) * kQ;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64, l16 = lane % 16, grp = lane / 16;

  // Tiles travel global -> registers -> LDS in two phases so that all of a thread's loads are in flight together
  // and the next tile's loads overlap the current tile's MFMAs.  Out-of-range elements read the slice's first
  // element (always present) and are replaced by zero on the way into LDS.
  constexpr int kPer = kKeys * kMaxD / 256;  // 32 elements of a K^T or V tile per thread
  float stage[kPer];
  uint32_t stage_ok = 0;
  const bool k_lanes_along_d = a.sKd <= a.sKn, v_lanes_along_d = a.sVd <= a.sVn;
  auto tile_index = [&](int i, bool along_d, int &n, int &k) {
    const int it = tid + i * 256;
    n = along_d ? it / kMaxD : it % kKeys;
    k = along_d ? it % kMaxD : it / kKeys;
  };
  auto load_k = [&](int c) {
    stage_ok = 0;
    if constexpr (VEC) {
#pragma unroll
      for (int i = 0; i < kPer / 4; ++i) {
        const int it = tid + i * 256, k = it / (kKeys / 4), n = it % (kKeys / 4) * 4;
        const bool ok = c * kKeys + n < a.Skv && k < a.D;
        const floatx4 x = *reinterpret_cast<const floatx4 *>(kt + off[2] + (ok ? k * a.sKd + c * kKeys + n : 0));
        stage[4 * i] = x.x, stage[4 * i + 1] = x.y, stage[4 * i + 2] = x.z, stage[4 * i + 3] = x.w;
        stage_ok |= static_cast<uint32_t>(ok) << i;
      }
    } else {
#pragma unroll
      for (int i = 0; i < kPer; ++i) {
        int n, k;
        tile_index(i, k_lanes_along_d, n, k);
        const bool ok = c * kKeys + n < a.Skv && k < a.D;
        stage[i] = kt[off[2] + (ok ? k * a.sKd + (c * kKeys + n) * a.sKn : 0)];
        stage_ok |= static_cast<uint32_t>(ok) << i;
      }
    }
  };
  auto load_v = [&](int c) {
    stage_ok = 0;
    if constexpr (VEC) {
#pragma unroll
      for (int i = 0; i < kPer / 4; ++i) {
        const int it = tid + i * 256, n = it / (kMaxD / 4), k = it % (kMaxD / 4) * 4;
        const bool ok = c * kKeys + n < a.Skv && k < a.D;
        const floatx4 x = *reinterpret_cast<const floatx4 *>(v + off[3] + (ok ? (c * kKeys + n) * a.sVn + k : 0));
        stage[4 * i] = x.x, stage[4 * i + 1] = x.y, stage[4 * i + 2] = x.z, stage[4 * i + 3] = x.w;
        stage_ok |= static_cast<uint32_t>(ok) << i;
      }
    } else {
#pragma unroll
      for (int i = 0; i < kPer; ++i) {
        int n, k;
        tile_index(i, v_lanes_along_d, n, k);
        const bool ok = c * kKeys + n < a.Skv && k < a.D;
        stage[i] = v[off[3] + (ok ? (c * kKeys + n) * a.sVn + k * a.sVd : 0)];
        stage_ok |= static_cast<uint32_t>(ok) << i;
      }
    }
  };
  auto store_stage = [&](bool along_d, bool transposed) {  // transposed: LDS [k][n] (K^T), else [n][k] (V)
    if constexpr (VEC) {
#pragma unroll
      for (int i = 0; i < kPer / 4; ++i) {
        const int it = tid + i * 256;
        const bool ok = stage_ok >> i & 1u;
        floatx4 x = {0.0f, 0.0f, 0.0f, 0.0f};
        if (ok) x = floatx4{stage[4 * i], stage[4 * i + 1], stage[4 * i + 2], stage[4 * i + 3]};
        float *dst = transposed ? kv + it / (kKeys / 4) * kLdK + it % (kKeys / 4) * 4
                                : kv + it / (kMaxD / 4) * kLdV + it % (kMaxD / 4) * 4;
        *reinterpret_cast<floatx4 *>(dst) = x;
      }
    } else {
#pragma unroll
      for (int i = 0; i < kPer; ++i) {
        int n, k;
        tile_index(i, along_d, n, k);
        kv[transposed ? k * kLdK + n : n * kLdV + k] = (stage_ok >> i & 1u) ? stage[i] : 0.0f;
      }
    }
  };

  // ---- Q block -> LDS [m][k], zero padded; the first K^T chunk is requested with it ------------------------
  {
    constexpr int kPerQ = kQ * kMaxD / 256;  // 4
    float qreg[kPerQ];
    if constexpr (VEC) {
      const int m = tid / (kMaxD / 4), k = tid % (kMaxD / 4) * 4;
      const bool ok = m0 + m < a.Sq && k < a.D;
      floatx4 x = *reinterpret_cast<const floatx4 *>(q + off[1] + (ok ? (m0 + m) * a.sQm + k : 0));
      if (!ok) x = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
      load_k(0);
      *reinterpret_cast<floatx4 *>(qs + m * kLdQ + k) = x;
    } else {
#pragma unroll
      for (int i = 0; i < kPerQ; ++i) {
        const int it = tid + i * 256, m = it / kMaxD, k = it % kMaxD;
        const bool ok = m0 + m < a.Sq && k < a.D;
        qreg[i] = q[off[1] + (ok ? (m0 + m) * a.sQm + k * a.sQd : 0)];
        if (!ok) qreg[i] = 0.0f;
      }
      load_k(0);
#pragma unroll
      for (int i = 0; i < kPerQ; ++i) {
        const int it = tid + i * 256;
        qs[(it / kMaxD) * kLdQ + it % kMaxD] = qreg[i];
      }
    }
  }
  // row-wise phase: lane handles query row tid / 16, keys [kNpt * (tid % 16), +kNpt); its mask and condition
  // values are requested now
  const int rw_row = tid / 16, rw_n0 = tid % 16 * kNpt;
  float mask_v[kNpt];
  uint32_t keep = ~0u;
  {
    const bool row_ok = m0 + rw_row < a.Sq;
    uint8_t cond_v[kNpt];
#pragma unroll
    for (int i = 0; i < kNpt; ++i) {
      const bool ok = row_ok && rw_n0 + i < a.Skv;
      mask_v[i] = mask != nullptr ? mask[off[4] + (ok ? (m0 + rw_row) * a.sMm + (rw_n0 + i) * a.sMn : 0)] : 0.0f;
      cond_v[i] = cond != nullptr ? cond[off[5] + (ok ? (m0 + rw_row) * a.sCm + (rw_n0 + i) * a.sCn : 0)] : uint8_t{1};
    }
    if (cond != nullptr) {
      keep = 0;
#pragma unroll
      for (int i = 0; i < kNpt; ++i) keep |= static_cast<uint32_t>(cond_v[i] != 0) << i;
    }
  }

  // ---- scores -> LDS strip ------------------------------------------------------------------------------
  // v_mfma_f32_16x16x4_f32: lane supplies A[m = lane % 16][k = lane / 16] and B[k = lane / 16][n = lane % 16] and
  // receives D[m = 4 * (lane / 16) + i][n = lane % 16], i = 0..3.  The k index is permuted so that lane group g
  // covers k = kk + 4 g + e in MFMA e: one 128-bit LDS read feeds four MFMAs.
  const int d16 = (a.D + 15) / 16 * 16;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    if (c > 0) __syncthreads();  // kv free
    store_stage(k_lanes_along_d, true);
    if (c + 1 < CHUNKS) load_k(c + 1);
    else load_v(0);
    __syncthreads();
    floatx4 s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int kk = 0; kk < d16; kk += 16) {
      const int kb = kk + 4 * grp;
      const floatx4 av = *reinterpret_cast<const floatx4 *>(qs + l16 * kLdQ + kb);
      const float a4[4] = {av.x, av.y, av.z, av.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[e], kv[(kb + e) * kLdK + wave * 32 + l16], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[e], kv[(kb + e) * kLdK + wave * 32 + 16 + l16], s1, 0, 0, 0);
      }
    }
    const float r0[4] = {s0.x, s0.y, s0.z, s0.w}, r1[4] = {s1.x, s1.y, s1.z, s1.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ps[(4 * grp + i) * kLdP + c * kKeys + wave * 32 + l16] = r0[i];
      ps[(4 * grp + i) * kLdP + c * kKeys + wave * 32 + 16 + l16] = r1[i];
    }
  }
  __syncthreads();  // the strip is complete, the last K^T chunk is consumed

  // ---- scale, mask, condition, row softmax (unnormalised) ------------------------------------------------
  {
    float x[kNpt];
#pragma unroll
    for (int i = 0; i < kNpt; i += 4) {
      const floatx4 t = *reinterpret_cast<const floatx4 *>(ps + rw_row * kLdP + rw_n0 + i);
      x[i] = t.x, x[i + 1] = t.y, x[i + 2] = t.z, x[i + 3] = t.w;
    }
    float mx = -__FLT_MAX__;
#pragma unroll
    for (int i = 0; i < kNpt; ++i) {
      float y = a.scale_is_divisor ? x[i] / a.scale : x[i] * a.scale;
      if (mask != nullptr) y = y + mask_v[i];
      if ((keep >> i & 1u) == 0) y = a.fill;
      if (rw_n0 + i >= a.Skv) y = -__FLT_MAX__;
      x[i] = y;
      mx = fmaxf(mx, y);
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < kNpt; ++i) {
      x[i] = rw_n0 + i < a.Skv ? expf(x[i] - mx) : 0.0f;
      sum += x[i];
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
#pragma unroll
    for (int i = 0; i < kNpt; i += 4) {
      *reinterpret_cast<floatx4 *>(ps + rw_row * kLdP + rw_n0 + i) = floatx4{x[i], x[i + 1], x[i + 2], x[i + 3]};
    }
    if (tid % 16 == 0) row_sum[rw_row] = sum;
  }

  // ---- out = (P . V) / row sum: wave w owns head columns [16 w, +16) --------------------------------------
  floatx4 o = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    if (c > 0) __syncthreads();  // kv free
    store_stage(v_lanes_along_d, false);  // V chunk -> LDS [key][d]
    if (c + 1 < CHUNKS) load_v(c + 1);
    __syncthreads();
    if (wave * 16 < a.D) {
#pragma unroll 4
      for (int kk = 0; kk < kKeys; kk += 16) {
        const int kb = kk + 4 * grp;
        const floatx4 av = *reinterpret_cast<const floatx4 *>(ps + l16 * kLdP + c * kKeys + kb);
        const float a4[4] = {av.x, av.y, av.z, av.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[e], kv[(kb + e) * kLdV + wave * 16 + l16], o, 0, 0, 0);
        }
      }
    }
  }
  {
    const float r[4] = {o.x, o.y, o.z, o.w};
    const int k = wave * 16 + l16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * grp + i;
      if (m0 + m < a.Sq && k < a.D) out[off[0] + (m0 + m) * a.sOm + k * a.sOd] = r[i] / row_sum[m];
    }
  }
}

}  // namespace
}  // namespace fl

using namespace fl;

extern "C" {

int fluidml_hip_attention(const fl_tensor *q, const fl_tensor *kt, const fl_tensor *v, const fl_tensor *out, double scale,
                          int32_t scale_is_divisor, const fl_tensor *add_mask, const fl_tensor *keep_cond, double fill,
                          void *stream) {
  FL_CHECK(CheckView(q));
  FL_CHECK(CheckView(kt));
  FL_CHECK(CheckView(v));
  FL_CHECK(CheckView(out));
  if (q->dtype != FL_FLOAT32 || kt->dtype != FL_FLOAT32 || v->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  const int rank = out->rank;
  if (rank < 2 || q->rank != rank || kt->rank != rank || v->rank != rank) return FL_ERR_RANK;
  AttentionArgs a;
  std::memset(&a, 0, sizeof(a));
  a.Sq = static_cast<int32_t>(q->shape[rank - 2]);
  a.D = static_cast<int32_t>(q->shape[rank - 1]);
  a.Skv = static_cast<int32_t>(kt->shape[rank - 1]);
  if (kt->shape[rank - 2] != a.D || v->shape[rank - 2] != a.Skv || v->shape[rank - 1] != a.D ||
      out->shape[rank - 2] != a.Sq || out->shape[rank - 1] != a.D) return FL_ERR_SHAPE;
  if (a.D > kMaxD || a.Skv > 2 * kKeys) return FL_ERR_UNSUPPORTED;
  a.sQm = static_cast<int32_t>(q->strides[rank - 2]);
  a.sQd = static_cast<int32_t>(q->strides[rank - 1]);
  a.sKd = static_cast<int32_t>(kt->strides[rank - 2]);
  a.sKn = static_cast<int32_t>(kt->strides[rank - 1]);
  a.sVn = static_cast<int32_t>(v->strides[rank - 2]);
  a.sVd = static_cast<int32_t>(v->strides[rank - 1]);
  a.sOm = static_cast<int32_t>(out->strides[rank - 2]);
  a.sOd = static_cast<int32_t>(out->strides[rank - 1]);
  a.scale = static_cast<float>(scale);
  a.scale_is_divisor = scale_is_divisor;
  a.fill = static_cast<float>(fill);
  // score-shaped index space [batch..., Sq, Skv] for the broadcast operands
  int64_t score_shape[kMaxRank], ms[kMaxRank] = {}, cs[kMaxRank] = {};
  for (int i = 0; i < rank - 2; ++i) score_shape[i] = out->shape[i];
  score_shape[rank - 2] = a.Sq;
  score_shape[rank - 1] = a.Skv;
  if (add_mask != nullptr) {
    FL_CHECK(CheckView(add_mask));
    if (add_mask->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    FL_CHECK(BroadcastStrides(add_mask, rank, score_shape, ms));
    a.sMm = static_cast<int32_t>(ms[rank - 2]);
    a.sMn = static_cast<int32_t>(ms[rank - 1]);
  }
  if (keep_cond != nullptr) {
    FL_CHECK(CheckView(keep_cond));
    if (keep_cond->dtype != FL_BOOL) return FL_ERR_DTYPE;
    FL_CHECK(BroadcastStrides(keep_cond, rank, score_shape, cs));
    a.sCm = static_cast<int32_t>(cs[rank - 2]);
    a.sCn = static_cast<int32_t>(cs[rank - 1]);
  }
  LoopNest nest;
  nest.n_operands = 6;
  nest.rank = rank - 2;
  int64_t n_batch = 1;
  for (int i = 0; i < rank - 2; ++i) {
    if (q->shape[i] != out->shape[i] || kt->shape[i] != out->shape[i] || v->shape[i] != out->shape[i]) return FL_ERR_SHAPE;
    nest.shape[i] = out->shape[i];
    nest.strides[0][i] = out->strides[i];
    nest.strides[1][i] = q->strides[i];
    nest.strides[2][i] = kt->strides[i];
    nest.strides[3][i] = v->strides[i];
    nest.strides[4][i] = ms[i];
    nest.strides[5][i] = cs[i];
    n_batch *= out->shape[i];
  }
  nest.Canonicalise();
  a.batch = MakeNestArgs<6>(nest);
  a.q_blocks = static_cast<uint32_t>((a.Sq + kQ - 1) / kQ);
  const int64_t blocks = n_batch * a.q_blocks;
  if (blocks > INT32_MAX) return FL_ERR_TOO_LARGE;
  if (blocks == 0 || a.D == 0) return FL_OK;
  if (a.Skv == 0) return FL_ERR_UNSUPPORTED;
  const dim3 grid(static_cast<uint32_t>(blocks)), block(256);
  float *o = static_cast<float *>(out->base);
  const float *qp = static_cast<const float *>(q->base), *kp = static_cast<const float *>(kt->base),
              *vp = static_cast<const float *>(v->base);
  const float *mp = add_mask ? static_cast<const float *>(add_mask->base) : nullptr;
  const uint8_t *cp = keep_cond ? static_cast<const uint8_t *>(keep_cond->base) : nullptr;
  auto mult4 = [](int64_t x) { return x % 4 == 0; };
  bool vec = a.sQd == 1 && a.sKn == 1 && a.sVd == 1 && a.D % 4 == 0 && a.Skv % 4 == 0 && mult4(a.sQm) && mult4(a.sKd) &&
             mult4(a.sVn) && reinterpret_cast<uintptr_t>(qp) % 16 == 0 && reinterpret_cast<uintptr_t>(kp) % 16 == 0 &&
             reinterpret_cast<uintptr_t>(vp) % 16 == 0;
  for (int i = 0; i < rank - 2; ++i) vec = vec && mult4(q->strides[i]) && mult4(kt->strides[i]) && mult4(v->strides[i]);
  if (a.Skv <= kKeys) {
    if (vec) FL_LAUNCH((AttentionKernel<1, true>), grid, block, 0, AsStream(stream), a, o, qp, kp, vp, mp, cp);
    else FL_LAUNCH((AttentionKernel<1, false>), grid, block, 0, AsStream(stream), a, o, qp, kp, vp, mp, cp);
  } else {
    if (vec) FL_LAUNCH((AttentionKernel<2, true>), grid, block, 0, AsStream(stream), a, o, qp, kp, vp, mp, cp);
    else FL_LAUNCH((AttentionKernel<2, false>), grid, block, 0, AsStream(stream), a, o, qp, kp, vp, mp, cp);
  }
  return LaunchStatus();
}

}  // extern "C"
