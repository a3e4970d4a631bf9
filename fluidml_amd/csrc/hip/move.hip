// Data-movement kernels whose index map is not a pure stride map (HBM bound):
// Reshape/Flatten (logical re-linearisation through two layouts), the three
// Gather variants plus the fused embedding sum, and CumSum.
// Reference: src/structure/kernel/kernel/{reshape,flatten,gather,gather_add_add,
// cum_sum}.cpp.
#include "fl_common.h"

namespace fl {

int StridedCopy(const fl_tensor *in, int64_t in_offset, const int64_t *in_strides, const fl_tensor *out,
                int64_t out_offset, int rank, const int64_t *shape, const int64_t *out_strides, void *stream);

namespace {

constexpr int kBlock = 256;

template <typename T, int N>
struct alignas(sizeof(T) * N) Vec {
  T v[N];
};

template <int NOPS>
__device__ __forceinline__ void ItemOffsets(const NestArgs<NOPS> &a, uint32_t item, int32_t *off) {
  int32_t acc[NOPS];
#pragma unroll
  for (int o = 0; o < NOPS; ++o) acc[o] = 0;
  a.AddOffsets(item, acc);
#pragma unroll
  for (int o = 0; o < NOPS; ++o) off[o] = acc[o];
}

// ---- Reshape ------------------------------------------------------------------

// nest operand 0: output physical offset, operand 1: logical linear index t.
// `src` holds the input's logical dims (merged where contiguous, never
// reordered) so t can be de-linearised into an input offset.
template <typename T>
__global__ __launch_bounds__(kBlock) void ReshapeKernel(NestArgs<2> a, NestArgs<1> src, uint32_t n,
                                                        T *__restrict__ out, const T *__restrict__ in) {
  const uint32_t item = blockIdx.x * kBlock + threadIdx.x;
  if (item >= n) return;
  int32_t off[2];
  ItemOffsets<2>(a, item, off);
  int32_t in_off[1] = {0};
  src.AddOffsets(static_cast<uint32_t>(off[1]), in_off);
  out[off[0]] = in[in_off[0]];
}

// Merge logically adjacent dims that are contiguous, keeping logical order.
void MergeLogical(const fl_tensor *t, LoopNest *nest) {
  nest->n_operands = 1;
  nest->rank = 0;
  for (int i = 0; i < t->rank; ++i) {
    if (t->shape[i] == 1) continue;
    if (nest->rank > 0 && nest->strides[0][nest->rank - 1] == t->strides[i] * t->shape[i]) {
      nest->shape[nest->rank - 1] *= t->shape[i];
      nest->strides[0][nest->rank - 1] = t->strides[i];
    } else {
      nest->shape[nest->rank] = t->shape[i];
      nest->strides[0][nest->rank] = t->strides[i];
      ++nest->rank;
    }
  }
  if (nest->rank == 0) {
    nest->rank = 1;
    nest->shape[0] = 1;
    nest->strides[0][0] = 0;
  }
}

int LogicalReshape(const fl_tensor *in, const fl_tensor *out, void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (in->dtype != out->dtype) return FL_ERR_DTYPE;
  const int64_t n = Numel(in);
  if (n != Numel(out)) return FL_ERR_SHAPE;
  LoopNest src;
  MergeLogical(in, &src);
  LoopNest dst;
  MergeLogical(out, &dst);
  if (src.rank == 1 && dst.rank == 1) {
    // both sides are one strided run in logical order: plain (vectorisable) copy
    return StridedCopy(in, 0, src.strides[0], out, 0, 1, &n, dst.strides[0], stream);
  }
  LoopNest nest;
  nest.rank = out->rank;
  nest.n_operands = 2;
  int64_t acc = 1;
  for (int i = out->rank - 1; i >= 0; --i) {
    nest.shape[i] = out->shape[i];
    nest.strides[0][i] = out->strides[i];
    nest.strides[1][i] = acc;
    acc *= out->shape[i];
  }
  nest.Canonicalise();
  NestArgs<2> a = MakeNestArgs<2>(nest);
  NestArgs<1> s = MakeNestArgs<1>(src);
  const uint32_t grid = static_cast<uint32_t>((n + kBlock - 1) / kBlock);
  hipStream_t st = AsStream(stream);
  switch (DtypeSize(in->dtype)) {
    case 1:
      FL_LAUNCH(ReshapeKernel<uint8_t>, dim3(grid), dim3(kBlock), 0, st, a, s, static_cast<uint32_t>(n),
                         static_cast<uint8_t *>(out->base), static_cast<const uint8_t *>(in->base));
      break;
    case 2:
      FL_LAUNCH(ReshapeKernel<uint16_t>, dim3(grid), dim3(kBlock), 0, st, a, s, static_cast<uint32_t>(n),
                         static_cast<uint16_t *>(out->base), static_cast<const uint16_t *>(in->base));
      break;
    case 4:
      FL_LAUNCH(ReshapeKernel<uint32_t>, dim3(grid), dim3(kBlock), 0, st, a, s, static_cast<uint32_t>(n),
                         static_cast<uint32_t *>(out->base), static_cast<const uint32_t *>(in->base));
      break;
    case 8:
      FL_LAUNCH(ReshapeKernel<uint64_t>, dim3(grid), dim3(kBlock), 0, st, a, s, static_cast<uint32_t>(n),
                         static_cast<uint64_t *>(out->base), static_cast<const uint64_t *>(in->base));
      break;
    default: return FL_ERR_DTYPE;
  }
  return LaunchStatus();
}

// ---- Gather ---------------------------------------------------------------------

// nest operands: 0 out, 1 indices, 2 data (all dims but the gathered one),
// 3 and 4 optional addends.  data element = data[off2 + idx * axis_stride].
template <typename T, int VEC, int NADD>
__global__ __launch_bounds__(kBlock) void GatherKernel(NestArgs<3 + NADD> a, uint32_t n_items, int32_t axis_stride,
                                                       int64_t axis_len, T *__restrict__ out,
                                                       const int64_t *__restrict__ indices, const T *__restrict__ data,
                                                       const T *__restrict__ add0, const T *__restrict__ add1) {
  const uint32_t item = blockIdx.x * kBlock + threadIdx.x;
  if (item >= n_items) return;
  int32_t off[3 + NADD];
  ItemOffsets<3 + NADD>(a, item, off);
  int64_t idx = indices[off[1]];
  if (idx < 0) idx += axis_len;           // ONNX negative indexing
  idx = idx < 0 ? 0 : (idx >= axis_len ? axis_len - 1 : idx);  // never read outside the table
  const T *src = data + off[2] + static_cast<int32_t>(idx) * axis_stride;
  if constexpr (VEC == 1) {
    T v = *src;
    if constexpr (NADD >= 1) v = v + add0[off[3]];
    if constexpr (NADD >= 2) v = v + add1[off[4]];
    out[off[0]] = v;
  } else {
    Vec<T, VEC> v = *reinterpret_cast<const Vec<T, VEC> *>(src);
    if constexpr (NADD >= 1) {
      const Vec<T, VEC> w = *reinterpret_cast<const Vec<T, VEC> *>(add0 + off[3]);
#pragma unroll
      for (int i = 0; i < VEC; ++i) v.v[i] = v.v[i] + w.v[i];
    }
    if constexpr (NADD >= 2) {
      const Vec<T, VEC> w = *reinterpret_cast<const Vec<T, VEC> *>(add1 + off[4]);
#pragma unroll
      for (int i = 0; i < VEC; ++i) v.v[i] = v.v[i] + w.v[i];
    }
    *reinterpret_cast<Vec<T, VEC> *>(out + off[0]) = v;
  }
}

template <typename T, int NADD>
int LaunchGather(LoopNest nest, int64_t axis_stride, int64_t axis_len, void *out, const void *indices,
                 const void *data, const void *add0, const void *add1, hipStream_t stream) {
  nest.Canonicalise();
  int64_t total = 1;
  for (int i = 0; i < nest.rank; ++i) total *= nest.shape[i];
  constexpr int kVec = 4;
  const int inner = nest.rank - 1;
  const void *ptrs[5] = {out, nullptr, data, add0, add1};
  bool vec_ok = nest.shape[inner] % kVec == 0 && nest.strides[1][inner] == 0 && axis_stride % kVec == 0;
  for (int o = 0; o < 3 + NADD && vec_ok; ++o) {
    if (o == 1) continue;
    if (nest.strides[o][inner] != 1 || !IsAligned(ptrs[o], sizeof(T) * kVec)) vec_ok = false;
    for (int d = 0; d < inner && vec_ok; ++d) {
      if (nest.strides[o][d] % kVec != 0) vec_ok = false;
    }
  }
  if (vec_ok) {
    nest.shape[inner] /= kVec;
    for (int o = 0; o < 3 + NADD; ++o) nest.strides[o][inner] *= kVec;
  }
  const int64_t n_items = vec_ok ? total / kVec : total;
  NestArgs<3 + NADD> a = MakeNestArgs<3 + NADD>(nest);
  const uint32_t grid = static_cast<uint32_t>((n_items + kBlock - 1) / kBlock);
  if (vec_ok) {
    FL_LAUNCH((GatherKernel<T, kVec, NADD>), dim3(grid), dim3(kBlock), 0, stream, a,
                       static_cast<uint32_t>(n_items), static_cast<int32_t>(axis_stride), axis_len,
                       static_cast<T *>(out), static_cast<const int64_t *>(indices), static_cast<const T *>(data),
                       static_cast<const T *>(add0), static_cast<const T *>(add1));
  } else {
    FL_LAUNCH((GatherKernel<T, 1, NADD>), dim3(grid), dim3(kBlock), 0, stream, a,
                       static_cast<uint32_t>(n_items), static_cast<int32_t>(axis_stride), axis_len,
                       static_cast<T *>(out), static_cast<const int64_t *>(indices), static_cast<const T *>(data),
                       static_cast<const T *>(add0), static_cast<const T *>(add1));
  }
  return LaunchStatus();
}

// out = data[..., indices[...], ...] with `indices` replacing `axis` of data.
int GatherNest(const fl_tensor *data, const fl_tensor *indices, const fl_tensor *out, int64_t axis, LoopNest *nest) {
  FL_CHECK(CheckView(data));
  FL_CHECK(CheckView(indices));
  FL_CHECK(CheckView(out));
  if (indices->dtype != FL_INT64) return FL_ERR_DTYPE;
  if (data->dtype != out->dtype) return FL_ERR_DTYPE;
  if (axis < 0 || axis >= data->rank) return FL_ERR_ATTR;
  if (out->rank != data->rank - 1 + indices->rank) return FL_ERR_RANK;
  nest->rank = out->rank;
  for (int i = 0; i < out->rank; ++i) {
    nest->shape[i] = out->shape[i];
    nest->strides[0][i] = out->strides[i];
    nest->strides[1][i] = 0;
    nest->strides[2][i] = 0;
    if (i < axis) {
      if (out->shape[i] != data->shape[i]) return FL_ERR_SHAPE;
      nest->strides[2][i] = data->strides[i];
    } else if (i < axis + indices->rank) {
      if (out->shape[i] != indices->shape[i - axis]) return FL_ERR_SHAPE;
      nest->strides[1][i] = indices->strides[i - axis];
    } else {
      const int j = i - indices->rank + 1;
      if (out->shape[i] != data->shape[j]) return FL_ERR_SHAPE;
      nest->strides[2][i] = data->strides[j];
    }
  }
  return FL_OK;
}

// ---- CumSum -------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(kBlock) void CumSumKernel(NestArgs<2> outer, uint32_t n_rows, uint32_t len, int32_t so,
                                                       int32_t si, T *__restrict__ out, const T *__restrict__ in) {
  const uint32_t row = blockIdx.x * kBlock + threadIdx.x;
  if (row >= n_rows) return;
  int32_t off[2];
  ItemOffsets<2>(outer, row, off);
  T acc = 0;
  for (uint32_t j = 0; j < len; ++j) {
    acc += in[off[1] + static_cast<int32_t>(j) * si];
    out[off[0] + static_cast<int32_t>(j) * so] = acc;
  }
}

// ---- Pad followed by steps that only re-address its result, as one copy ---------------------------------
// out[i0, i1, ..] = padded[view_offset + sum(i_k * view_strides[k])] where `padded` is the Pad's output taken as a
// dense row-major tensor that is never written: the element is read from the Pad's input when it lies in the
// interior and is zero otherwise.  (ConvBERT unfolds the values of its span-based convolution this way: Pad along
// the sequence, a Gather of sliding windows, Transpose, Reshape.)
struct PadViewArgs {
  int32_t out_rank, pad_rank;
  uint32_t n;
  int32_t view_offset;
  FastDiv out_div[kMaxRank];      // out logical extents
  int32_t out_strides[kMaxRank];
  int32_t view_strides[kMaxRank];
  FastDiv pad_div[kMaxRank];      // padded extents
  int32_t before[kMaxRank];       // padding in front, per dim
  int32_t src_shape[kMaxRank], src_strides[kMaxRank];
};

__global__ __launch_bounds__(kBlock) void PadViewCopyKernel(PadViewArgs a, uint32_t *__restrict__ out,
                                                            const uint32_t *__restrict__ src) {
  const uint32_t idx = blockIdx.x * kBlock + threadIdx.x;
  if (idx >= a.n) return;
  uint32_t rem = idx;
  int32_t out_off = 0, lin = a.view_offset;
#pragma unroll
  for (int d = kMaxRank - 1; d >= 0; --d) {
    if (d < a.out_rank) {
      uint32_t q, r;
      a.out_div[d].DivMod(rem, q, r);
      rem = q;
      out_off += static_cast<int32_t>(r) * a.out_strides[d];
      lin += static_cast<int32_t>(r) * a.view_strides[d];
    }
  }
  uint32_t left = static_cast<uint32_t>(lin);
  int32_t src_off = 0;
  bool inside = true;
#pragma unroll
  for (int d = kMaxRank - 1; d >= 0; --d) {
    if (d < a.pad_rank) {
      uint32_t q, r;
      a.pad_div[d].DivMod(left, q, r);
      left = q;
      const int32_t c = static_cast<int32_t>(r) - a.before[d];
      inside = inside && static_cast<uint32_t>(c) < static_cast<uint32_t>(a.src_shape[d]);
      src_off += c * a.src_strides[d];
    }
  }
  out[out_off] = inside ? src[src_off] : 0u;
}

int PadViewCopy(const fl_tensor *in, const int64_t *pads_before, const int64_t *padded_shape, int32_t n_dims,
                int64_t view_offset, const int64_t *view_strides, const fl_tensor *out, void *stream) {
  if (!in || !pads_before || !padded_shape || !view_strides || !out) return FL_ERR_NULL;
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (in->dtype != out->dtype) return FL_ERR_DTYPE;
  if (DtypeSize(in->dtype) != 4) return FL_ERR_UNSUPPORTED;
  if (n_dims != in->rank) return FL_ERR_RANK;
  PadViewArgs a;
  std::memset(&a, 0, sizeof(a));
  int64_t padded_numel = 1;
  for (int d = 0; d < in->rank; ++d) {
    if (pads_before[d] < 0 || padded_shape[d] < pads_before[d] + in->shape[d]) return FL_ERR_ATTR;
    padded_numel *= padded_shape[d];
    a.pad_div[d] = FastDiv(static_cast<uint32_t>(padded_shape[d]));
    a.before[d] = static_cast<int32_t>(pads_before[d]);
    a.src_shape[d] = static_cast<int32_t>(in->shape[d]);
    a.src_strides[d] = static_cast<int32_t>(in->strides[d]);
  }
  const int64_t n = Numel(out);
  if (n == 0) return FL_OK;
  if (padded_numel > 0x7fffffff || n > 0x7fffffff || view_offset < 0) return FL_ERR_TOO_LARGE;
  int64_t last = view_offset;
  for (int d = 0; d < out->rank; ++d) {
    if (view_strides[d] < 0 || view_strides[d] > 0x7fffffff) return FL_ERR_ATTR;
    last += (out->shape[d] - 1) * view_strides[d];
    a.out_div[d] = FastDiv(static_cast<uint32_t>(out->shape[d]));
    a.out_strides[d] = static_cast<int32_t>(out->strides[d]);
    a.view_strides[d] = static_cast<int32_t>(view_strides[d]);
  }
  if (last >= padded_numel) return FL_ERR_SHAPE;  // the view reaches outside the padded tensor
  a.out_rank = out->rank;
  a.pad_rank = in->rank;
  a.n = static_cast<uint32_t>(n);
  a.view_offset = static_cast<int32_t>(view_offset);
  FL_LAUNCH(PadViewCopyKernel, dim3(static_cast<uint32_t>((n + kBlock - 1) / kBlock)), dim3(kBlock), 0, AsStream(stream), a,
            static_cast<uint32_t *>(out->base), static_cast<const uint32_t *>(in->base));
  return LaunchStatus();
}

}  // namespace
}  // namespace fl

using namespace fl;

extern "C" {

int fluidml_hip_pad_view_copy(const fl_tensor *in, const int64_t *pads_before, const int64_t *padded_shape, int32_t n_dims,
                              int64_t view_offset, const int64_t *view_strides, const fl_tensor *out, void *stream) {
  return PadViewCopy(in, pads_before, padded_shape, n_dims, view_offset, view_strides, out, stream);
}

int fluidml_hip_reshape(const fl_tensor *in, const fl_tensor *out, void *stream) {
  return LogicalReshape(in, out, stream);
}

int fluidml_hip_flatten(const fl_tensor *in, const fl_tensor *out, int64_t axis, void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (out->rank != 2) return FL_ERR_RANK;
  if (axis < 0) axis += in->rank;
  if (axis < 0 || axis > in->rank) return FL_ERR_ATTR;
  int64_t d0 = 1, d1 = 1;
  for (int i = 0; i < in->rank; ++i) (i < axis ? d0 : d1) *= in->shape[i];
  if (out->shape[0] != d0 || out->shape[1] != d1) return FL_ERR_SHAPE;
  return LogicalReshape(in, out, stream);
}

int fluidml_hip_gather_constant_indices_tensor(const fl_tensor *in, const fl_tensor *indices, const fl_tensor *out,
                                               int64_t axis, void *stream) {
  LoopNest nest;
  nest.n_operands = 3;
  if (!in || !indices || !out) return FL_ERR_NULL;
  FL_CHECK(GatherNest(in, indices, out, axis, &nest));
  hipStream_t s = AsStream(stream);
  switch (DtypeSize(in->dtype)) {
    case 4:
      return LaunchGather<uint32_t, 0>(nest, in->strides[axis], in->shape[axis], out->base, indices->base, in->base,
                                       nullptr, nullptr, s);
    case 8:
      return LaunchGather<uint64_t, 0>(nest, in->strides[axis], in->shape[axis], out->base, indices->base, in->base,
                                       nullptr, nullptr, s);
    default: return FL_ERR_DTYPE;
  }
}

int fluidml_hip_gather_constant_data_tensor(const fl_tensor *indices, const fl_tensor *data, const fl_tensor *out,
                                            void *stream) {
  LoopNest nest;
  nest.n_operands = 3;
  if (!indices || !data || !out) return FL_ERR_NULL;
  FL_CHECK(GatherNest(data, indices, out, 0, &nest));
  if (data->dtype != FL_FLOAT32) return FL_ERR_DTYPE;  // reference gather.cpp:224-233
  return LaunchGather<float, 0>(nest, data->strides[0], data->shape[0], out->base, indices->base, data->base, nullptr,
                                nullptr, AsStream(stream));
}

int fluidml_hip_gather_constant_data_tensor_add(const fl_tensor *indices, const fl_tensor *data, const fl_tensor *add0,
                                                const fl_tensor *out, void *stream) {
  LoopNest nest;
  nest.n_operands = 4;
  if (!indices || !data || !add0 || !out) return FL_ERR_NULL;
  FL_CHECK(GatherNest(data, indices, out, 0, &nest));
  FL_CHECK(CheckView(add0));
  if (data->dtype != FL_FLOAT32 || add0->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  FL_CHECK(BroadcastStrides(add0, out->rank, out->shape, nest.strides[3]));
  return LaunchGather<float, 1>(nest, data->strides[0], data->shape[0], out->base, indices->base, data->base,
                                add0->base, nullptr, AsStream(stream));
}

int fluidml_hip_gather_constant_data_tensor_add_tensor_lhs_add_tensor_lhs(const fl_tensor *indices,
                                                                          const fl_tensor *data, const fl_tensor *add0,
                                                                          const fl_tensor *add1, const fl_tensor *out,
                                                                          void *stream) {
  LoopNest nest;
  nest.n_operands = 5;
  if (!indices || !data || !add0 || !add1 || !out) return FL_ERR_NULL;
  FL_CHECK(GatherNest(data, indices, out, 0, &nest));
  FL_CHECK(CheckView(add0));
  FL_CHECK(CheckView(add1));
  if (data->dtype != FL_FLOAT32 || add0->dtype != FL_FLOAT32 || add1->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  FL_CHECK(BroadcastStrides(add0, out->rank, out->shape, nest.strides[3]));
  FL_CHECK(BroadcastStrides(add1, out->rank, out->shape, nest.strides[4]));
  // a broadcast addend along the innermost dim defeats the vector path; the
  // scalar path handles it
  return LaunchGather<float, 2>(nest, data->strides[0], data->shape[0], out->base, indices->base, data->base,
                                add0->base, add1->base, AsStream(stream));
}

int fluidml_hip_cum_sum(const fl_tensor *in, const fl_tensor *out, int64_t axis, void *stream) {
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(out));
  if (!SameShape(in, out)) return FL_ERR_SHAPE;
  if (in->dtype != out->dtype) return FL_ERR_DTYPE;
  if (axis < 0 || axis >= in->rank) return FL_ERR_ATTR;
  LoopNest nest;
  nest.n_operands = 2;
  for (int i = 0; i < in->rank; ++i) {
    if (i == axis) continue;
    nest.shape[nest.rank] = in->shape[i];
    nest.strides[0][nest.rank] = out->strides[i];
    nest.strides[1][nest.rank] = in->strides[i];
    ++nest.rank;
  }
  nest.Canonicalise();
  int64_t rows = 1;
  for (int i = 0; i < nest.rank; ++i) rows *= nest.shape[i];
  NestArgs<2> a = MakeNestArgs<2>(nest);
  const uint32_t grid = static_cast<uint32_t>((rows + kBlock - 1) / kBlock);
  hipStream_t s = AsStream(stream);
  const uint32_t len = static_cast<uint32_t>(in->shape[axis]);
  const int32_t so = static_cast<int32_t>(out->strides[axis]), si = static_cast<int32_t>(in->strides[axis]);
  if (in->dtype == FL_INT64) {
    FL_LAUNCH(CumSumKernel<int64_t>, dim3(grid), dim3(kBlock), 0, s, a, static_cast<uint32_t>(rows), len, so,
                       si, static_cast<int64_t *>(out->base), static_cast<const int64_t *>(in->base));
  } else if (in->dtype == FL_INT32) {
    FL_LAUNCH(CumSumKernel<int32_t>, dim3(grid), dim3(kBlock), 0, s, a, static_cast<uint32_t>(rows), len, so,
                       si, static_cast<int32_t *>(out->base), static_cast<const int32_t *>(in->base));
  } else {
    return FL_ERR_DTYPE;  // reference cum_sum.cpp uses arith.addi only
  }
  return LaunchStatus();
}

}  // extern "C"
