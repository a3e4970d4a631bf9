/*
 * TEST INFRASTRUCTURE -- not part of the product.
 *
 * CPU restatement of the loop nests FluidML's kernels emit as linalg.generic /
 * affine.for (reference src/structure/kernel/kernel/ *.cpp), over the same strided
 * views the product's C ABI takes.  Each function walks the iteration space in
 * the order the reference's lowering does (linalg -> affine loops, dimension 0
 * outermost; reference src/worker/lower.cpp:38-46), keeps partial sums in the
 * output / scratch memory as fp32 exactly where the reference does, and uses
 * separate multiply and add (build with -ffp-contract=off: the reference
 * pipeline sets no contraction flag).
 *
 * Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may
 * load this file's library; the product never does.
 *
 * What pins each function is recorded in tests/test_oracle_kernels.py
 * (numpy/torch closed forms on the reference's own node-test shapes,
 * reference test/python/node/ *.py).
 *
 * `flags` bits are those of include/fluidml_hip.h (FL_REF_*): a set bit makes
 * the function follow the reference literally where it departs from ONNX.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#include "../include/fluidml_hip.h"

typedef fl_tensor view;

static int64_t numel(const view *t) {
  int64_t n = 1;
  for (int i = 0; i < t->rank; ++i) n *= t->shape[i];
  return n;
}

/* advance a row-major multi-index; returns 0 when it wraps */
static int next_index(int rank, const int64_t *shape, int64_t *idx) {
  for (int d = rank - 1; d >= 0; --d) {
    if (++idx[d] < shape[d]) return 1;
    idx[d] = 0;
  }
  return 0;
}

static int64_t offset_of(const view *t, const int64_t *idx) {
  int64_t off = 0;
  for (int i = 0; i < t->rank; ++i) off += idx[i] * t->strides[i];
  return off;
}

/* offset of `t` for output index `idx` of rank `rank` under trailing-aligned
 * broadcast: equal dim -> d_i, dim 1 -> 0 (reference utils.cpp:16-52) */
static int64_t bcast_offset(const view *t, int rank, const int64_t *idx) {
  int64_t off = 0;
  for (int i = 0; i < rank; ++i) {
    const int j = t->rank - rank + i;
    if (j >= 0 && t->shape[j] != 1) off += idx[i] * t->strides[j];
  }
  return off;
}

#define F32(t) ((float *)(t)->base)
#define CF32(t) ((const float *)(t)->base)

/* ---- elementwise, float32 unary ------------------------------------------- */

enum {
  OP_ADD_C, OP_RSUB_C, OP_MUL_C, OP_DIV_C, OP_POW_C, OP_ERF, OP_RELU, OP_CLIP,
  OP_TANH, OP_SQRT, OP_NEG, OP_COPY
};

static float maximumf_(float a, float b) { /* arith.maximumf: NaN propagates */
  if (a != a) return a;
  if (b != b) return b;
  return a > b ? a : b;
}
static float minimumf_(float a, float b) {
  if (a != a) return a;
  if (b != b) return b;
  return a < b ? a : b;
}

/* add.cpp:22-79, sub.cpp:16-67, mul.cpp:19-54, div.cpp:18-66, pow.cpp:15-61,
 * erf.cpp:18-45, relu.cpp:12-46, clip.cpp:13-48, tanh.cpp:12-40,
 * sqrt.cpp:13-36, neg.cpp:17-40, dropout.cpp:13-33: identity maps, all-parallel */
int oracle_unary_f32(int op, const view *in, const view *out, double c0, double c1) {
  int64_t idx[FL_MAX_RANK] = {0};
  const float a = (float)c0, b = (float)c1;
  if (numel(out) == 0) return 0;
  do {
    const float x = CF32(in)[offset_of(in, idx)];
    float y;
    switch (op) {
      case OP_ADD_C: y = x + a; break;
      case OP_RSUB_C: y = a - x; break;
      case OP_MUL_C: y = x * a; break;
      case OP_DIV_C: y = x / a; break;
      case OP_POW_C: y = powf(x, a); break;
      case OP_ERF: y = erff(x); break;
      case OP_RELU: y = maximumf_(x, 0.0f); break;
      case OP_CLIP: y = minimumf_(maximumf_(x, a), b); break;
      case OP_TANH: y = tanhf(x); break;
      case OP_SQRT: y = sqrtf(x); break;
      case OP_NEG: y = -x; break;
      case OP_COPY: y = x; break;
      default: return -1;
    }
    F32(out)[offset_of(out, idx)] = y;
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* AddConstantKernel integer forms (add.cpp:29-44), CastKernel (cast.cpp:12-63),
 * EqualKernel (equal.cpp:14-51), NotKernel (not.cpp:11-41) */
static int64_t load_int(const view *t, int64_t off) {
  switch (t->dtype) {
    case FL_BOOL: return ((const uint8_t *)t->base)[off];
    case FL_INT32: return ((const int32_t *)t->base)[off];
    case FL_INT64: return ((const int64_t *)t->base)[off];
    default: return 0;
  }
}
static void store_int(const view *t, int64_t off, int64_t v) {
  switch (t->dtype) {
    case FL_BOOL: ((uint8_t *)t->base)[off] = (uint8_t)(v & 1); break;
    case FL_INT32: ((int32_t *)t->base)[off] = (int32_t)v; break; /* arith.trunci */
    case FL_INT64: ((int64_t *)t->base)[off] = v; break;
    default: break;
  }
}
enum { IOP_ADD_C, IOP_CAST, IOP_EQ_C, IOP_NOT };
int oracle_unary_int(int op, const view *in, const view *out, double c) {
  int64_t idx[FL_MAX_RANK] = {0};
  do {
    const int64_t x = load_int(in, offset_of(in, idx));
    int64_t y;
    switch (op) {
      case IOP_ADD_C: y = x + (int64_t)c; break;
      case IOP_CAST: y = x; break; /* bool source is 0/1: zero extension */
      case IOP_EQ_C: y = x == (int64_t)c; break;
      case IOP_NOT: y = x ^ 1; break;
      default: return -1;
    }
    store_int(out, offset_of(out, idx), y);
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* ---- elementwise, binary with broadcast -------------------------------------- */
enum { BOP_ADD, BOP_SUB, BOP_MUL, BOP_DIV };
/* add.cpp:83-125, sub.cpp:71-99, mul.cpp:56-99, div.cpp:70-105 */
int oracle_binary_f32(int op, const view *lhs, const view *rhs, const view *out) {
  int64_t idx[FL_MAX_RANK] = {0};
  do {
    const float a = CF32(lhs)[bcast_offset(lhs, out->rank, idx)];
    const float b = CF32(rhs)[bcast_offset(rhs, out->rank, idx)];
    float y;
    switch (op) {
      case BOP_ADD: y = a + b; break;
      case BOP_SUB: y = a - b; break;
      case BOP_MUL: y = a * b; break;
      case BOP_DIV: y = a / b; break;
      default: return -1;
    }
    F32(out)[offset_of(out, idx)] = y;
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}
/* MulCommonKernel integer form (mul.cpp:78-84) */
int oracle_mul_int(const view *lhs, const view *rhs, const view *out) {
  int64_t idx[FL_MAX_RANK] = {0};
  do {
    const int64_t a = load_int(lhs, bcast_offset(lhs, out->rank, idx));
    const int64_t b = load_int(rhs, bcast_offset(rhs, out->rank, idx));
    store_int(out, offset_of(out, idx), a * b);
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* where.cpp:30-80 (y scalar: y_tensor == NULL) and :90-150 (y tensor) */
int oracle_where(const view *cond, const view *x, const view *y_tensor, double y_scalar, const view *out) {
  int64_t idx[FL_MAX_RANK] = {0};
  do {
    const uint8_t c = ((const uint8_t *)cond->base)[bcast_offset(cond, out->rank, idx)];
    const float xv = CF32(x)[bcast_offset(x, out->rank, idx)];
    const float yv = y_tensor ? CF32(y_tensor)[bcast_offset(y_tensor, out->rank, idx)] : (float)y_scalar;
    F32(out)[offset_of(out, idx)] = c ? xv : yv;
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* add_div_erf_add_mul_mul.cpp:29-132 */
int oracle_add_div_erf_add_mul_mul(const view *in, const view *add0, const view *out, double div, double add1,
                                   double mul1) {
  int64_t idx[FL_MAX_RANK] = {0};
  const float cd = (float)div, ca = (float)add1, cm = (float)mul1;
  do {
    const float x = CF32(in)[bcast_offset(in, out->rank, idx)];
    const float b = CF32(add0)[bcast_offset(add0, out->rank, idx)];
    const float add0_op = x + b;
    const float div_op = add0_op / cd;
    const float erf_op = erff(div_op);
    const float add1_op = erf_op + ca;
    const float mul0_op = add0_op * add1_op;
    F32(out)[offset_of(out, idx)] = mul0_op * cm;
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* unsqueeze_sub_mul.cpp:19-69: out[i...] = (sub - in[non-axis i...]) * mul */
int oracle_unsqueeze_sub_mul(const view *in, const view *out, const int64_t *axes, int32_t n_axes, double sub,
                             double mul) {
  int64_t idx[FL_MAX_RANK] = {0};
  do {
    int64_t off = 0;
    int j = 0;
    for (int i = 0; i < out->rank; ++i) {
      int is_axis = 0;
      for (int k = 0; k < n_axes; ++k) {
        const int64_t ax = axes[k] < 0 ? axes[k] + out->rank : axes[k];
        if (ax == i) is_axis = 1;
      }
      if (!is_axis) off += idx[i] * in->strides[j++];
    }
    F32(out)[offset_of(out, idx)] = ((float)sub - CF32(in)[off]) * (float)mul;
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* ---- data movement ---------------------------------------------------------------- */

static size_t dtype_size(int32_t dtype) {
  switch (dtype) {
    case FL_BOOL: return 1;
    case FL_FLOAT16: return 2;
    case FL_INT32: case FL_FLOAT32: return 4;
    default: return 8;
  }
}

static void copy_elem(const view *dst, int64_t doff, const view *src, int64_t soff) {
  const size_t esz = dtype_size(src->dtype);
  memcpy((char *)dst->base + doff * (int64_t)esz, (const char *)src->base + soff * (int64_t)esz, esz);
}

/* transpose.cpp:19-48: input map identity, output map (d_perm[0], d_perm[1], ...) */
int oracle_transpose(const view *in, const view *out, const int64_t *perm) {
  int64_t idx[FL_MAX_RANK] = {0}, oidx[FL_MAX_RANK];
  do {
    for (int i = 0; i < out->rank; ++i) oidx[i] = idx[perm[i]];
    copy_elem(out, offset_of(out, oidx), in, offset_of(in, idx));
  } while (next_index(in->rank, in->shape, idx));
  return 0;
}

/* reshape.cpp:18-64: t in [0,N): both sides de-linearised in logical row-major order.
 * flatten.cpp:15-63 builds the same map for a rank-2 output. */
int oracle_reshape(const view *in, const view *out) {
  const int64_t n = numel(in);
  for (int64_t t = 0; t < n; ++t) {
    int64_t ioff = 0, ooff = 0, prod = n;
    for (int i = 0; i < in->rank; ++i) {
      const int64_t r = t % prod;
      prod /= in->shape[i];
      ioff += (r / prod) * in->strides[i];
    }
    prod = n;
    for (int i = 0; i < out->rank; ++i) {
      const int64_t r = t % prod;
      prod /= out->shape[i];
      ooff += (r / prod) * out->strides[i];
    }
    copy_elem(out, ooff, in, ioff);
  }
  return 0;
}

/* squeeze.cpp:17-54: input map has constant 0 at squeezed axes */
int oracle_squeeze(const view *in, const view *out, const int64_t *axes, int32_t n_axes) {
  int64_t idx[FL_MAX_RANK] = {0};
  do {
    int64_t off = 0;
    int j = 0;
    for (int i = 0; i < in->rank; ++i) {
      int squeezed = 0;
      for (int k = 0; k < n_axes; ++k)
        if ((axes[k] < 0 ? axes[k] + in->rank : axes[k]) == i) squeezed = 1;
      if (!squeezed) off += idx[j++] * in->strides[i];
    }
    copy_elem(out, offset_of(out, idx), in, off);
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* unsqueeze.cpp:20-63: input map drops the axes' loop dims */
int oracle_unsqueeze(const view *in, const view *out, const int64_t *axes, int32_t n_axes) {
  int64_t idx[FL_MAX_RANK] = {0};
  do {
    int64_t off = 0;
    int j = 0;
    for (int i = 0; i < out->rank; ++i) {
      int is_axis = 0;
      for (int k = 0; k < n_axes; ++k)
        if ((axes[k] < 0 ? axes[k] + out->rank : axes[k]) == i) is_axis = 1;
      if (!is_axis) off += idx[i] * in->strides[j++];
    }
    copy_elem(out, offset_of(out, idx), in, off);
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* slice.cpp:17-55: subview(offsets, out shape, steps) copied to out */
int oracle_slice(const view *in, const view *out, const int64_t *starts, const int64_t *axes, const int64_t *steps,
                 int32_t n) {
  int64_t offs[FL_MAX_RANK] = {0}, step[FL_MAX_RANK];
  for (int i = 0; i < in->rank; ++i) step[i] = 1;
  for (int k = 0; k < n; ++k) {
    offs[axes[k]] = starts[k];
    step[axes[k]] = steps[k];
  }
  int64_t idx[FL_MAX_RANK] = {0};
  do {
    int64_t off = 0;
    for (int i = 0; i < in->rank; ++i) off += (offs[i] + idx[i] * step[i]) * in->strides[i];
    copy_elem(out, offset_of(out, idx), in, off);
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* concat.cpp:18-68: lhs into out[0:lhs], rhs into out[lhs:] along axis */
int oracle_concat2(const view *lhs, const view *rhs, const view *out, int64_t axis) {
  int64_t idx[FL_MAX_RANK] = {0};
  do {
    copy_elem(out, offset_of(out, idx), lhs, offset_of(lhs, idx));
  } while (next_index(lhs->rank, lhs->shape, idx));
  memset(idx, 0, sizeof(idx));
  do {
    copy_elem(out, offset_of(out, idx) + lhs->shape[axis] * out->strides[axis], rhs, offset_of(rhs, idx));
  } while (next_index(rhs->rank, rhs->shape, idx));
  return 0;
}

/* pad.cpp:15-51: input copied into the interior; the border is left as it was */
int oracle_pad(const view *in, const view *out, const int64_t *pads_before, uint32_t flags) {
  int64_t idx[FL_MAX_RANK] = {0};
  int64_t base = 0;
  if (!(flags & FL_REF_PAD_BORDER_UNWRITTEN)) {
    /* ONNX constant mode with value 0: every output element starts as zero */
    const size_t esz = dtype_size(out->dtype);
    do {
      memset((char *)out->base + offset_of(out, idx) * (int64_t)esz, 0, esz);
    } while (next_index(out->rank, out->shape, idx));
  }
  for (int i = 0; i < in->rank; ++i) base += pads_before[i] * out->strides[i];
  do {
    copy_elem(out, base + offset_of(out, idx), in, offset_of(in, idx));
  } while (next_index(in->rank, in->shape, idx));
  return 0;
}

/* gather.cpp:100-139.  The data map compares loop positions with the raw
 * `axis` attribute (:116); FL_REF_GATHER_RAW_AXIS keeps that, otherwise the
 * axis is normalised first. */
int oracle_gather_index_scalar(const view *in, const view *out, int64_t axis, int64_t index, uint32_t flags) {
  int64_t ax = axis;
  if (!(flags & FL_REF_GATHER_RAW_AXIS) && ax < 0) ax += in->rank;
  if (ax < 0) return -1; /* raw negative axis: no position matches, map is ill-formed */
  int64_t idx[FL_MAX_RANK] = {0};
  do {
    int64_t off = 0;
    for (int i = 0; i < in->rank; ++i) {
      if (i == ax) off += index * in->strides[i];
      else off += idx[i < ax ? i : i - 1] * in->strides[i];
    }
    copy_elem(out, offset_of(out, idx), in, off);
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* gather.cpp:24-86,149-186: out[o0..o_{axis-1}, i..., rest] = in[o0.., indices[i...], rest] */
int oracle_gather_indices_tensor(const view *in, const view *indices, const view *out, int64_t axis) {
  int64_t idx[FL_MAX_RANK] = {0};
  const int ir = indices->rank;
  do {
    int64_t ioff = 0;
    for (int i = 0; i < ir; ++i) ioff += idx[axis + i] * indices->strides[i];
    const int64_t g = ((const int64_t *)indices->base)[ioff];
    int64_t off = 0;
    for (int i = 0; i < axis; ++i) off += idx[i] * in->strides[i];
    off += g * in->strides[axis];
    for (int i = (int)axis + ir; i < out->rank; ++i) off += idx[i] * in->strides[i - ir + 1];
    copy_elem(out, offset_of(out, idx), in, off);
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* gather.cpp:195-272 (axis 0 of a constant table) and gather_add_add.cpp:25-163
 * (table[ids] + add0 + add1, evaluated in that order; add0/add1 may be NULL) */
int oracle_gather_data_tensor(const view *indices, const view *data, const view *add0, const view *add1,
                              const view *out) {
  int64_t idx[FL_MAX_RANK] = {0};
  const int ir = indices->rank;
  do {
    int64_t ioff = 0;
    for (int i = 0; i < ir; ++i) ioff += idx[i] * indices->strides[i];
    const int64_t g = ((const int64_t *)indices->base)[ioff];
    int64_t off = g * data->strides[0];
    for (int i = ir; i < out->rank; ++i) off += idx[i] * data->strides[i - ir + 1];
    float v = CF32(data)[off];
    if (add0) v = v + CF32(add0)[bcast_offset(add0, out->rank, idx)];
    if (add1) v = v + CF32(add1)[bcast_offset(add1, out->rank, idx)];
    F32(out)[offset_of(out, idx)] = v;
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* cum_sum.cpp:53-87: loops with `axis` moved innermost, running integer sum */
int oracle_cum_sum(const view *in, const view *out, int64_t axis) {
  int64_t shape[FL_MAX_RANK], idx[FL_MAX_RANK] = {0}, real[FL_MAX_RANK];
  const int rank = in->rank;
  for (int i = 0; i < rank; ++i) shape[i] = in->shape[i];
  { const int64_t t = shape[axis]; shape[axis] = shape[rank - 1]; shape[rank - 1] = t; }
  int64_t acc = 0;
  do {
    if (idx[rank - 1] == 0) acc = 0;
    for (int i = 0; i < rank; ++i) real[i] = idx[i];
    { const int64_t t = real[axis]; real[axis] = real[rank - 1]; real[rank - 1] = t; }
    acc += load_int(in, offset_of(in, real));
    store_int(out, offset_of(out, real), acc);
  } while (next_index(rank, shape, idx));
  return 0;
}

/* ---- row reductions ------------------------------------------------------------------ */

/* offset into the dense scratch tensor of shape(in) with axis -> 1 */
static int64_t scratch_offset(const view *in, int64_t axis, const int64_t *idx) {
  int64_t off = 0;
  for (int i = 0; i < in->rank; ++i) {
    if (i == axis) continue;
    int64_t stride = 1;
    for (int j = i + 1; j < in->rank; ++j) stride *= (j == axis ? 1 : in->shape[j]);
    off += idx[i] * stride;
  }
  return off;
}

/* softmax.cpp:22-139: the six passes, through `scratch` */
int oracle_softmax(const view *in, const view *out, float *scratch, int64_t axis) {
  int64_t idx[FL_MAX_RANK] = {0};
  int64_t rows = numel(in) / in->shape[axis];
  for (int64_t r = 0; r < rows; ++r) scratch[r] = -3.402823466e+38f; /* numeric_limits<float>::lowest() */
  do { /* arith.maxnumf(input, value) */
    const float x = CF32(in)[offset_of(in, idx)];
    float *m = &scratch[scratch_offset(in, axis, idx)];
    *m = fmaxf(x, *m);
  } while (next_index(in->rank, in->shape, idx));
  do {
    F32(out)[offset_of(out, idx)] = CF32(in)[offset_of(in, idx)] - scratch[scratch_offset(in, axis, idx)];
  } while (next_index(in->rank, in->shape, idx));
  do {
    float *o = &F32(out)[offset_of(out, idx)];
    *o = expf(*o);
  } while (next_index(in->rank, in->shape, idx));
  for (int64_t r = 0; r < rows; ++r) scratch[r] = 0.0f;
  do {
    scratch[scratch_offset(in, axis, idx)] += F32(out)[offset_of(out, idx)];
  } while (next_index(in->rank, in->shape, idx));
  do {
    float *o = &F32(out)[offset_of(out, idx)];
    *o = *o / scratch[scratch_offset(in, axis, idx)];
  } while (next_index(in->rank, in->shape, idx));
  return 0;
}

/* layer_normalization.cpp:33-220.  The first accumulation adds onto whatever
 * `scratch` holds (no fill before :126); a caller that wants the ONNX result
 * passes zeroed scratch. */
int oracle_layer_norm(const view *in, const view *scale, const view *bias, const view *out, float *scratch,
                      int64_t axis, double epsilon) {
  int64_t idx[FL_MAX_RANK] = {0};
  const int64_t rows = numel(in) / in->shape[axis];
  const float n = (float)in->shape[axis], eps = (float)epsilon;
  do {
    scratch[scratch_offset(in, axis, idx)] += CF32(in)[offset_of(in, idx)];
  } while (next_index(in->rank, in->shape, idx));
  for (int64_t r = 0; r < rows; ++r) scratch[r] = scratch[r] / n;
  do {
    F32(out)[offset_of(out, idx)] = CF32(in)[offset_of(in, idx)] - scratch[scratch_offset(in, axis, idx)];
  } while (next_index(in->rank, in->shape, idx));
  for (int64_t r = 0; r < rows; ++r) scratch[r] = 0.0f;
  do {
    const float d = F32(out)[offset_of(out, idx)];
    float *v = &scratch[scratch_offset(in, axis, idx)];
    *v = *v + d * d;
  } while (next_index(in->rank, in->shape, idx));
  for (int64_t r = 0; r < rows; ++r) scratch[r] = scratch[r] / n;
  do {
    float *o = &F32(out)[offset_of(out, idx)];
    const float var = scratch[scratch_offset(in, axis, idx)];
    const float g = CF32(scale)[bcast_offset(scale, in->rank, idx)];
    const float b = CF32(bias)[bcast_offset(bias, in->rank, idx)];
    const float inv = 1.0f / sqrtf(var + eps);
    *o = (*o * inv) * g + b;
  } while (next_index(in->rank, in->shape, idx));
  return 0;
}

/* reduce_mean.cpp:16-98 (keepdims = 1) */
int oracle_reduce_mean(const view *in, const view *out, const int64_t *axes, int32_t n_axes) {
  int64_t idx[FL_MAX_RANK] = {0}, oidx[FL_MAX_RANK];
  int64_t divisor = 1;
  for (int k = 0; k < n_axes; ++k) divisor *= in->shape[axes[k]];
  do {
    F32(out)[offset_of(out, idx)] = 0.0f;
  } while (next_index(out->rank, out->shape, idx));
  do {
    for (int i = 0; i < in->rank; ++i) oidx[i] = idx[i];
    for (int k = 0; k < n_axes; ++k) oidx[axes[k]] = 0;
    float *o = &F32(out)[offset_of(out, oidx)];
    *o = CF32(in)[offset_of(in, idx)] + *o;
  } while (next_index(in->rank, in->shape, idx));
  do {
    float *o = &F32(out)[offset_of(out, idx)];
    *o = *o / (float)divisor;
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* maxpool.cpp:17-82 / averagepool.cpp:19-87: fold of the K subviews in
 * GenAllIndicesInOrder (row-major) order */
int oracle_pool(int is_max, const view *in, const view *out, const int64_t *kernel_shape, const int64_t *strides,
                int32_t n) {
  int64_t idx[FL_MAX_RANK] = {0}, kidx[FL_MAX_RANK];
  const int batches = in->rank - n;
  int64_t ksize = 1;
  for (int i = 0; i < n; ++i) ksize *= kernel_shape[i];
  do {
    float acc = 0.0f;
    memset(kidx, 0, sizeof(kidx));
    int first = 1;
    do {
      int64_t off = 0;
      for (int i = 0; i < in->rank; ++i) {
        if (i < batches) off += idx[i] * in->strides[i];
        else off += (kidx[i - batches] + idx[i] * strides[i - batches]) * in->strides[i];
      }
      const float v = CF32(in)[off];
      if (first) { acc = v; first = 0; }
      else acc = is_max ? maximumf_(acc, v) : acc + v;
    } while (next_index(n, kernel_shape, kidx));
    F32(out)[offset_of(out, idx)] = is_max ? acc : acc / (float)ksize;
  } while (next_index(out->rank, out->shape, idx));
  return 0;
}

/* ---- contractions ----------------------------------------------------------------------- */

/* matmul.cpp:28-59 with utils.cpp:64-147: fill 0, then (batch..., i, j, k)
 * accumulating into the output memory.  The six loop orders of `axes_` give
 * the same per-element k-ascending sum, so only (i,j,k) is restated. */
int oracle_matmul(const view *lhs, const view *rhs, const view *out) {
  const int r = out->rank;
  int64_t idx[FL_MAX_RANK] = {0};
  const int64_t M = out->shape[r - 2], N = out->shape[r - 1], K = lhs->shape[lhs->rank - 1];
  int64_t bshape[FL_MAX_RANK];
  for (int i = 0; i < r - 2; ++i) bshape[i] = out->shape[i];
  do {
    F32(out)[offset_of(out, idx)] = 0.0f;
  } while (next_index(r, out->shape, idx));
  memset(idx, 0, sizeof(idx));
  do {
    int64_t lo = 0, ro = 0, oo = 0;
    for (int i = 0; i < r - 2; ++i) {
      const int li = lhs->rank - r + i, ri = rhs->rank - r + i;
      if (li >= 0 && lhs->shape[li] != 1) lo += idx[i] * lhs->strides[li];
      if (ri >= 0 && rhs->shape[ri] != 1) ro += idx[i] * rhs->strides[ri];
      oo += idx[i] * out->strides[i];
    }
    const int64_t sAm = lhs->strides[lhs->rank - 2], sAk = lhs->strides[lhs->rank - 1];
    const int64_t sBk = rhs->strides[rhs->rank - 2], sBn = rhs->strides[rhs->rank - 1];
    const int64_t sCm = out->strides[r - 2], sCn = out->strides[r - 1];
    for (int64_t i = 0; i < M; ++i)
      for (int64_t j = 0; j < N; ++j) {
        float *o = &F32(out)[oo + i * sCm + j * sCn];
        for (int64_t k = 0; k < K; ++k) {
          const float mul = CF32(lhs)[lo + i * sAm + k * sAk] * CF32(rhs)[ro + k * sBk + j * sBn];
          *o = mul + *o;
        }
      }
  } while (r > 2 && next_index(r - 2, bshape, idx));
  return 0;
}

/* gemm.cpp:39-182: fill 0; out += A(transA) . B(transB); then
 * out = alpha * bias + beta * out (FL_REF_GEMM_SWAPPED_SCALARS, :176-179) or
 * out = alpha * out + beta * bias (ONNX). */
int oracle_gemm(const view *lhs, const view *rhs, const view *bias, const view *out, double alpha, double beta,
                int trans_a, int trans_b, uint32_t flags) {
  const int64_t M = out->shape[0], N = out->shape[1];
  const int64_t K = trans_a ? lhs->shape[0] : lhs->shape[1];
  const int64_t sAm = lhs->strides[trans_a ? 1 : 0], sAk = lhs->strides[trans_a ? 0 : 1];
  const int64_t sBk = rhs->strides[trans_b ? 1 : 0], sBn = rhs->strides[trans_b ? 0 : 1];
  const float a = (float)alpha, b = (float)beta;
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) F32(out)[i * out->strides[0] + j * out->strides[1]] = 0.0f;
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      float *o = &F32(out)[i * out->strides[0] + j * out->strides[1]];
      for (int64_t k = 0; k < K; ++k) {
        const float mul = CF32(lhs)[i * sAm + k * sAk] * CF32(rhs)[k * sBk + j * sBn];
        *o = mul + *o;
      }
    }
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      float *o = &F32(out)[i * out->strides[0] + j * out->strides[1]];
      const float bv = bias->rank == 1 ? CF32(bias)[j * bias->strides[0]]
                                       : CF32(bias)[i * bias->strides[0] + j * bias->strides[1]];
      if (flags & FL_REF_GEMM_SWAPPED_SCALARS) *o = a * bv + b * *o;
      else *o = a * *o + b * bv;
    }
  return 0;
}

/* conv.cpp:27-201 (+ :230-280 for padding).  Loop nest n, f, c, o..., k...
 * (group == 1) or n, f, o..., k... (depthwise), accumulating into the output;
 * then the bias pass.  With padding the reference convolves a zero-padded copy
 * of the input; reading 0 for out-of-range taps is the same arithmetic.
 *   FL_REF_CONV_UNIT_STRIDE : input index is o + k (strides/dilations unused, :71,:118)
 *   FL_REF_CONV_BIAS_INDEX1 : every element gets bias[1] (:181-182)            */
int oracle_conv(const view *in, const view *w, const view *bias, const view *out, const int64_t *pads,
                const int64_t *strides, const int64_t *dilations, int64_t group, uint32_t flags) {
  const int rank = out->rank, ns = rank - 2;
  const int64_t C = in->shape[1];
  const int depthwise = group != 1;
  int64_t idx[FL_MAX_RANK] = {0}, kidx[FL_MAX_RANK], kshape[FL_MAX_RANK];
  for (int d = 0; d < ns; ++d) kshape[d] = w->shape[2 + d];
  do {
    F32(out)[offset_of(out, idx)] = 0.0f;
  } while (next_index(rank, out->shape, idx));
  const int64_t c_loops = depthwise ? 1 : C;
  for (int64_t n = 0; n < out->shape[0]; ++n)
    for (int64_t f = 0; f < out->shape[1]; ++f)
      for (int64_t c = 0; c < c_loops; ++c) {
        int64_t oidx[FL_MAX_RANK] = {0};
        do {
          int64_t ooff = n * out->strides[0] + f * out->strides[1];
          for (int d = 0; d < ns; ++d) ooff += oidx[d] * out->strides[2 + d];
          float *o = &F32(out)[ooff];
          memset(kidx, 0, sizeof(kidx));
          do {
            int64_t ioff = n * in->strides[0] + (depthwise ? f : c) * in->strides[1];
            int64_t woff = f * w->strides[0] + c * w->strides[1];
            int inside = 1;
            for (int d = 0; d < ns; ++d) {
              const int64_t st = (flags & FL_REF_CONV_UNIT_STRIDE) || !strides ? 1 : strides[d];
              const int64_t di = (flags & FL_REF_CONV_UNIT_STRIDE) || !dilations ? 1 : dilations[d];
              const int64_t pos = oidx[d] * st + kidx[d] * di - (pads ? pads[d] : 0);
              if (pos < 0 || pos >= in->shape[2 + d]) inside = 0;
              ioff += pos * in->strides[2 + d];
              woff += kidx[d] * w->strides[2 + d];
            }
            const float x = inside ? CF32(in)[ioff] : 0.0f;
            const float mul = x * CF32(w)[woff];
            *o = mul + *o;
          } while (next_index(ns, kshape, kidx));
        } while (next_index(ns, out->shape + 2, oidx));
      }
  if (bias) {
    memset(idx, 0, sizeof(idx));
    do {
      float *o = &F32(out)[offset_of(out, idx)];
      const float bv = (flags & FL_REF_CONV_BIAS_INDEX1) ? CF32(bias)[1 * bias->strides[0]]
                                                         : CF32(bias)[idx[1] * bias->strides[0]];
      *o = bv + *o;
    } while (next_index(rank, out->shape, idx));
  }
  return 0;
}
