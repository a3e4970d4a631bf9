/*
 * fluidml_hip.h -- C ABI of the MI355X (gfx950) execution backend for FluidML.
 *
 * One entry point per FluidML kernel class (the strings returned by
 * `GetKernelName()`, reference include/structure/kernel/kernel/ *.h).  Where the
 * reference kernel's `Run(mlir::OpBuilder&, mlir::Value&...)` *emits* a
 * linalg.generic over strided memrefs, the entry point here *launches* a HIP
 * kernel over strided device views.  An `fl_tensor` carries exactly what the
 * reference kernels read from a `mlir::MemRefType`: element type, shape and
 * element strides (reference src/worker/builder.cpp:234-270 builds those
 * memrefs from the region's layout).
 *
 * Conventions
 *   - every pointer inside an fl_tensor is a DEVICE pointer to logical element
 *     (0,...,0); strides are in elements and may describe any permutation
 *     layout produced by utils::GenStrides (reference src/utils/utils.cpp:85-102);
 *   - `stream` is a hipStream_t passed as void*; NULL = the null stream;
 *   - every call is asynchronous on `stream` and returns 0 on success, a
 *     negative FL_ERR_* code for a rejected argument (nothing is launched) or a
 *     positive hipError_t from the runtime;
 *   - `scratch` is the node's buffer of the memory plan (reference
 *     flow::Node::GetBufferSize, src/structure/flow/node.cpp:500-519, 972-985,
 *     1355-1368).  The plan keeps those bytes so offsets stay identical to the
 *     reference; kernels that do not need them ignore the pointer;
 *   - `flags` selects literal reproduction of reference behaviours that differ
 *     from ONNX semantics (FL_REF_* below). 0 = ONNX semantics.
 *
 * No torch types, no C++ types: this header compiles as C.
 */
#ifndef FLUIDML_HIP_H_
#define FLUIDML_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FL_MAX_RANK 8

/* Element types; numbering follows `enum class Type` (reference
 * include/utils/type.h:11-19) so a host `Type` casts straight through. */
enum fl_dtype {
  FL_UNKNOWN = 0,
  FL_BOOL = 1, /* 1 byte, values 0/1 (sizeof(bool), reference src/utils/type.cpp:45) */
  FL_INT32 = 2,
  FL_INT64 = 3,
  FL_FLOAT16 = 4, /* carried, never computed on */
  FL_FLOAT32 = 5,
  FL_FLOAT64 = 6
};

enum fl_error {
  FL_OK = 0,
  FL_ERR_NULL = -1,        /* a required pointer is NULL */
  FL_ERR_RANK = -2,        /* rank outside [0, FL_MAX_RANK] or ranks inconsistent */
  FL_ERR_SHAPE = -3,       /* shapes do not satisfy the kernel's contract */
  FL_ERR_DTYPE = -4,       /* element type combination the reference leaves unreachable */
  FL_ERR_ATTR = -5,        /* attribute out of range (axis, pads, strides, ...) */
  FL_ERR_TOO_LARGE = -6,   /* more than 2^31-1 elements or offsets in one view */
  FL_ERR_SCRATCH = -7,     /* scratch smaller than the kernel needs */
  FL_ERR_UNSUPPORTED = -8, /* legal in ONNX, unreachable in the reference, not built */
  FL_ERR_STATIC_SCRATCH = -9 /* the launch needs more split-K workspace than the fixed
                              * FL_NO_ALLOC_SCRATCH_BYTES of fluidml_hip_matmul_no_alloc */
};

/* Literal-reference switches (each cites the reference lines it reproduces). */
enum fl_ref_flags {
  /* Conv reads input at o+k: `strides`/`dilations` never applied
   * (reference src/structure/kernel/kernel/conv.cpp:71,118). */
  FL_REF_CONV_UNIT_STRIDE = 1 << 0,
  /* Conv adds bias[1] to every output element (affine map is the constant 1,
   * reference conv.cpp:181-182). */
  FL_REF_CONV_BIAS_INDEX1 = 1 << 1,
  /* LayerNormalization accumulates the row sum on top of whatever the scratch
   * holds (first FillOp comes after the mean pass, reference
   * layer_normalization.cpp:126 vs :165). */
  FL_REF_LN_STALE_SCRATCH = 1 << 2,
  /* Gemm computes alpha*bias + beta*(A.B) (reference gemm.cpp:176-179);
   * without the flag: alpha*(A.B) + beta*bias as ONNX defines it. */
  FL_REF_GEMM_SWAPPED_SCALARS = 1 << 3,
  /* GatherConstantIndexScalar compares against the un-normalised axis
   * (reference gather.cpp:116). */
  FL_REF_GATHER_RAW_AXIS = 1 << 4,
  /* Pad copies the input into the interior and never writes the border, which
   * keeps whatever the arena held (reference pad.cpp:33-51 writes through a
   * subview only); without the flag the border is written as zero. */
  FL_REF_PAD_BORDER_UNWRITTEN = 1 << 5,
  /* Host side only (no kernel reads it): a constant tensor whose layout is not the default one is written as
   * data[row-major position of i] = values[strided position of i] and then read through those same strides (reference
   * src/worker/builder.cpp:290-297, :311-318); without the flag the element lands at its strided position. */
  FL_REF_CONSTANT_GATHERED = 1 << 6
};

/* Options of the contraction entry points (MatMul, Gemm, Conv with group 1).  The fused
 * entry points take them as their `flags`; the entry points whose `flags` carry
 * fl_ref_flags take them shifted left by FL_CONTRACT_SHIFT in the same word. */
enum fl_contract_flags {
  /* operands rounded to bf16 (nearest even), fp32 accumulation on the matrix
   * cores: the opt-in reduced-precision path; its error is reported separately
   * by bench.py.  Launches that do not run on the matrix cores ignore it
   * (at most 8 rows against k-contiguous weights: the weights are streamed in
   * fp32; depthwise and 3-d convolutions: the direct kernel). */
  FL_CONTRACT_BF16 = 1 << 0,
  /* fluidml_hip_conv_chain_scale_add only: `addend` multiplies the value instead of being added to it (a MulCommon
   * behind the convolution, reference mul.cpp) */
  FL_CONTRACT_ADDEND_IS_FACTOR = 1 << 1
  /* bits 4..7: enum fl_contract_tile; bits 8..13: number of workgroups that share
   * the K range of a tile (FL_CONTRACT_TILE / FL_CONTRACT_SPLITS below) */
};
#define FL_CONTRACT_SHIFT 16

/* Tile configurations of the contraction kernel (MatMul, Gemm).  The reference's
 * generators time the six loop orders of their kernel and keep the fastest
 * (src/structure/kernel/generator/matmul.cpp:88-131, gemm.cpp:106-151); on this
 * backend the choice that matters is the workgroup's tile and how many
 * workgroups share the K range of a tile.  FL_TILE_RULE / 0 splits leave either
 * to the library's own rule.  A configuration that does not exist for the operands of
 * a call (the direct-to-LDS ones need both operands on their 128-bit load path and K a
 * multiple of the chunk; a split needs that many K chunks and room in the
 * stream's workspace) makes the call return FL_ERR_UNSUPPORTED with nothing
 * launched, so a tuner can simply try them all.  Every configuration gives the
 * same result from run to run; different configurations add the products in
 * different orders. */
enum fl_contract_tile {
  FL_TILE_RULE = 0,
  FL_TILE_32x32_STAGED = 1, /* 32x32 tile, four waves split K, tiles staged through registers by four more waves */
  FL_TILE_64x64_STAGED = 2, /* 64x64 tile, 2x2 waves, four K chunks in flight in registers */
  FL_TILE_32x32_K4 = 3,     /* the following load tiles from global memory straight into LDS: */
  FL_TILE_64x32_K2 = 4,     /*   64x32 tile, two waves side by side times two K slices */
  FL_TILE_64x64 = 5,        /*   64x64 tile, 2x2 waves */
  FL_TILE_64x64_K2 = 6,     /*   64x64 tile, 2x2 waves times two K slices (eight waves) */
  FL_TILE_128x64 = 7,       /*   128x64 tile, 4x2 waves */
  FL_TILE_128x128_STAGED = 8, /* bf16 operands only: 128x128 tile, 2x2 waves with 2x2 accumulators each, four K chunks in flight */
  FL_TILE_COUNT = 9
};
#define FL_CONTRACT_TILE_SHIFT 4
#define FL_CONTRACT_SPLIT_SHIFT 8
#define FL_CONTRACT_MAX_SPLITS 63
#define FL_CONTRACT_TILE(tile) ((uint32_t)(tile) << FL_CONTRACT_TILE_SHIFT)
#define FL_CONTRACT_SPLITS(n) ((uint32_t)(n) << FL_CONTRACT_SPLIT_SHIFT)

/* A short chain of elementwise operations on one float32 value, used by the
 * launch-level fusions below.  Step i replaces v (initially the chain's input
 * x) by op[i](v, c[i]) or op[i](v, x); every operation is the one the
 * standalone kernel of that name performs. */
enum fl_ew_op {
  FL_EW_ADD_C = 0, /* v + c   (AddConstantKernel) */
  FL_EW_RSUB_C,    /* c - v   (SubConstantLhsKernel) */
  FL_EW_MUL_C,     /* v * c   (MulConstantKernel) */
  FL_EW_DIV_C,     /* v / c   (DivConstantRhsKernel) */
  FL_EW_POW_C,     /* powf(v, c) (PowKernel) */
  FL_EW_ERF,       /* ErfKernel */
  FL_EW_RELU,      /* ReluKernel (NaN propagates) */
  FL_EW_TANH,      /* TanhKernel */
  FL_EW_SQRT,      /* SqrtKernel */
  FL_EW_NEG,       /* NegKernel */
  FL_EW_ADD_X,     /* v + x   (AddCommonKernel with the chain input) */
  FL_EW_MUL_X,     /* v * x   (MulCommonKernel) */
  FL_EW_SUB_X,     /* v - x   (SubCommonKernel, chain value on the left) */
  FL_EW_RSUB_X,    /* x - v */
  FL_EW_DIV_X,     /* v / x   (DivCommonKernel, chain value on the left) */
  FL_EW_RDIV_X     /* x / v */
};
#define FL_EW_MAX_STEPS 8
typedef struct fl_ew_program {
  int32_t n; /* 0..FL_EW_MAX_STEPS */
  int32_t op[FL_EW_MAX_STEPS];
  float c[FL_EW_MAX_STEPS];
} fl_ew_program;

typedef struct fl_tensor {
  void *base;
  int32_t dtype; /* enum fl_dtype */
  int32_t rank;
  int64_t shape[FL_MAX_RANK];
  int64_t strides[FL_MAX_RANK]; /* in elements */
} fl_tensor;

/* ------------------------------------------------------------------------- */
/* Library / device plumbing (replaces the MLIR ExecutionEngine + the per-call
 * host arena of reference src/worker/runner.cpp:56-120).                     */

/* Version of this ABI; bumped on any signature change (2: `flags` of the fused Gemm and Conv entry points;
 * 3: tile configuration and K splits in the contraction flags). */
int fluidml_hip_abi_version(void);
/* Human-readable text for a return code of this library (static storage). */
const char *fluidml_hip_error_string(int code);
/* Number of visible devices, or a negative/positive error code. */
int fluidml_hip_device_count(void);
/* Name and arch of device `dev` into caller buffers (NUL-terminated). */
int fluidml_hip_device_info(int dev, char *name, size_t name_len, char *arch,
                            size_t arch_len, int *compute_units,
                            size_t *total_mem);

/* One HBM arena of `bytes` bytes (reference runner.cpp:87-96 allocates
 * `FuncAttr::GetBuffer()` zeroed host bytes per Invoke; here it is allocated
 * once, zero-filled once, and lives until destroy). */
int fluidml_hip_arena_create(size_t bytes, void **arena);
int fluidml_hip_arena_destroy(void *arena);
int fluidml_hip_arena_zero(void *arena, size_t bytes, void *stream);
/* Constants (reference builder.cpp:273-361 embeds them as memref.global):
 * allocate device memory and copy `bytes` host bytes into it. */
int fluidml_hip_upload_constant(const void *host, size_t bytes, void **device);
int fluidml_hip_free(void *device);
int fluidml_hip_memcpy_h2d(void *device, const void *host, size_t bytes, void *stream);
int fluidml_hip_memcpy_d2h(void *host, const void *device, size_t bytes, void *stream);
int fluidml_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
int fluidml_hip_stream_create(void **stream);
int fluidml_hip_stream_destroy(void *stream);
int fluidml_hip_stream_synchronize(void *stream);
/* Event pair timing used by KernelEval::GetTimeCost (reference
 * src/evaluation/eval.cpp:64-100 times one JIT run with the host clock). */
int fluidml_hip_event_create(void **event);
int fluidml_hip_event_destroy(void *event);
int fluidml_hip_event_record(void *event, void *stream);
/* Work issued to `stream` after this call waits for what `event` recorded (the edge between the two branches of a
 * launch plan that runs an independent run of launches beside another; the reference runs its nodes one after the
 * other, runner.cpp:101-109).  Also valid while `event`'s stream is being captured: `stream` then joins the capture. */
int fluidml_hip_stream_wait_event(void *stream, void *event);
int fluidml_hip_event_elapsed_ns(void *start, void *stop, double *ns);
/* Kernel-exact timing for the calling thread: until cleared with (NULL, NULL),
 * every kernel an entry point below launches stamps `start`/`stop` with the
 * dispatch's own begin and end, so their elapsed time excludes launch latency
 * and queue gaps (what eval.cpp:64-100 cannot separate on the CPU).  If one call
 * launches several kernels the events describe the last one.  Not for use
 * during launch-plan capture. */
int fluidml_hip_time_kernels(void *start, void *stop);
/* Measurement helper without a counterpart in the reference: `waves_per_simd` (1 or 2) waves on every SIMD of the
 * current device each issue `count` dependent v_mfma_f32_32x32x2_f32 and nothing else.  `ns`: the median wave's
 * duration on the 100 MHz wall clock; `shader_ticks`: the same interval in shader clock ticks (one such instruction
 * occupies a SIMD's matrix pipe for 64 of them).  What a contraction kernel can reach at best on this device at the
 * clock it actually runs at: 4096 * count flops per wave in `ns`.  Allocates and frees a small device buffer. */
int fluidml_hip_mfma_rate(int32_t waves_per_simd, int32_t count, double *ns, double *shader_ticks);
/* Launch-plan capture: the node sequence of one Invoke recorded once and
 * replayed (the counterpart of re-running `_mlir_ciface_<name>`,
 * reference runner.cpp:101-109). */
int fluidml_hip_graph_begin_capture(void *stream);
int fluidml_hip_graph_end_capture(void *stream, void **graph_exec);
int fluidml_hip_graph_launch(void *graph_exec, void *stream);
int fluidml_hip_graph_destroy(void *graph_exec);

/* ------------------------------------------------------------------------- */
/* a.3 Elementwise kernels (HBM bound).                                       */
/* Scalar operands arrive as double, as the reference stores them
 * (`float64_t value_`, include/structure/flow/node.h:147-165), and are cast to
 * the tensor's element type inside the call.                                 */

/* AddConstantKernel: out = in + value; int32/int64/float32
 * (reference add.cpp:22-79). */
int fluidml_hip_add_constant(const fl_tensor *in, const fl_tensor *out, double value, void *stream);
/* AddCommonKernel: out = lhs + rhs with trailing-aligned broadcast
 * (reference add.cpp:83-125, utils.cpp:16-52). */
int fluidml_hip_add_common(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream);
/* SubConstantLhsKernel: out = value - in (reference sub.cpp:16-67). */
int fluidml_hip_sub_constant_lhs(const fl_tensor *in, const fl_tensor *out, double value, void *stream);
/* SubCommonKernel (reference sub.cpp:71-99). */
int fluidml_hip_sub_common(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream);
/* MulConstantKernel: out = in * value, float32 (reference mul.cpp:19-54). */
int fluidml_hip_mul_constant(const fl_tensor *in, const fl_tensor *out, double value, void *stream);
/* MulCommonKernel: integer or float (reference mul.cpp:56-99). */
int fluidml_hip_mul_common(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream);
/* DivConstantRhsKernel: out = in / value, true division (reference div.cpp:18-66). */
int fluidml_hip_div_constant_rhs(const fl_tensor *in, const fl_tensor *out, double value, void *stream);
/* DivCommonKernel (reference div.cpp:70-105). */
int fluidml_hip_div_common(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream);
/* PowKernel: out = powf(in, exponent) (reference pow.cpp:15-61). */
int fluidml_hip_pow(const fl_tensor *in, const fl_tensor *out, double exponent, void *stream);
/* ErfKernel (reference erf.cpp:18-45). */
int fluidml_hip_erf(const fl_tensor *in, const fl_tensor *out, void *stream);
/* ReluKernel (reference relu.cpp:12-46). */
int fluidml_hip_relu(const fl_tensor *in, const fl_tensor *out, void *stream);
/* ClipKernel: min(max(x, lo), hi) (reference clip.cpp:13-48). */
int fluidml_hip_clip(const fl_tensor *in, const fl_tensor *out, float lo, float hi, void *stream);
/* TanhKernel (reference tanh.cpp:12-40). */
int fluidml_hip_tanh(const fl_tensor *in, const fl_tensor *out, void *stream);
/* SqrtKernel (reference sqrt.cpp:13-36). */
int fluidml_hip_sqrt(const fl_tensor *in, const fl_tensor *out, void *stream);
/* NegKernel (reference neg.cpp:17-40). */
int fluidml_hip_neg(const fl_tensor *in, const fl_tensor *out, void *stream);
/* NotKernel: bool xor 1 (reference not.cpp:11-41). */
int fluidml_hip_not(const fl_tensor *in, const fl_tensor *out, void *stream);
/* CastKernel: integer<->integer; bool zero-extends (reference cast.cpp:12-63). */
int fluidml_hip_cast(const fl_tensor *in, const fl_tensor *out, void *stream);
/* EqualKernel: int64 == value -> bool (reference equal.cpp:14-51). */
int fluidml_hip_equal(const fl_tensor *in, const fl_tensor *out, double value, void *stream);
/* DropoutKernel: identity copy (reference dropout.cpp:13-33). */
int fluidml_hip_dropout(const fl_tensor *in, const fl_tensor *out, void *stream);
/* WhereConstantCondConstantScalarYKernel: out = cond ? x : y
 * (reference where.cpp:30-80); cond is a bool tensor broadcast to out. */
int fluidml_hip_where_constant_cond_constant_scalar_y(const fl_tensor *cond, const fl_tensor *x, const fl_tensor *out, double y, void *stream);
/* WhereConstantCondConstantTensorYKernel (reference where.cpp:90-150). */
int fluidml_hip_where_constant_cond_constant_tensor_y(const fl_tensor *cond, const fl_tensor *x, const fl_tensor *y, const fl_tensor *out, void *stream);
/* AddDivErfAddMulMulKernel: t = x + b; out = t * (erf(t / div) + add1) * mul1
 * (reference add_div_erf_add_mul_mul.cpp:29-132). */
int fluidml_hip_add_div_erf_add_mul_mul(const fl_tensor *in, const fl_tensor *add0, const fl_tensor *out, double div, double add1, double mul1, void *stream);
/* UnsqueezeSubLhsScalarMulRhsScalarKernel: out = (sub - unsqueeze(x)) * mul
 * (reference unsqueeze_sub_mul.cpp:19-69). */
int fluidml_hip_unsqueeze_sub_lhs_scalar_mul_rhs_scalar(const fl_tensor *in, const fl_tensor *out, const int64_t *axes, int32_t n_axes, double sub, double mul, void *stream);

/* ------------------------------------------------------------------------- */
/* a.4 Data-movement kernels (HBM bound).                                     */

/* TransposeKernel: out[d[perm[0]],...] = in[d0,...] (reference transpose.cpp:19-48). */
int fluidml_hip_transpose(const fl_tensor *in, const fl_tensor *out, const int64_t *perm, int32_t n_perm, void *stream);
/* ReshapeKernel: logical row-major reshape through both layouts
 * (reference reshape.cpp:18-64). */
int fluidml_hip_reshape(const fl_tensor *in, const fl_tensor *out, void *stream);
/* FlattenKernel (reference flatten.cpp:15-63). */
int fluidml_hip_flatten(const fl_tensor *in, const fl_tensor *out, int64_t axis, void *stream);
/* SqueezeKernel / UnsqueezeKernel (reference squeeze.cpp:17-54, unsqueeze.cpp:20-63). */
int fluidml_hip_squeeze(const fl_tensor *in, const fl_tensor *out, const int64_t *axes, int32_t n_axes, void *stream);
int fluidml_hip_unsqueeze(const fl_tensor *in, const fl_tensor *out, const int64_t *axes, int32_t n_axes, void *stream);
/* SliceKernel: per sliced axis (start, axis, step); extent = out shape
 * (reference slice.cpp:17-55). */
int fluidml_hip_slice(const fl_tensor *in, const fl_tensor *out, const int64_t *starts, const int64_t *axes, const int64_t *steps, int32_t n, void *stream);
/* Concat2Kernel (reference concat.cpp:18-68). */
int fluidml_hip_concat2(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, int64_t axis, void *stream);
/* PadKernel: input copied into the interior, border written as zero (ONNX
 * constant mode, value 0); with FL_REF_PAD_BORDER_UNWRITTEN only the interior
 * is written (reference pad.cpp:15-51). `pads_before[i]` per dimension. */
int fluidml_hip_pad(const fl_tensor *in, const fl_tensor *out, const int64_t *pads_before, int32_t n, uint32_t flags, void *stream);
/* PadKernel followed by kernels that only re-address its result (Gather with sliding-window indices, Slice,
 * Transpose, Reshape, ...) as ONE copy (reference pad.cpp:15-51, gather.cpp, transpose.cpp, reshape.cpp): the padded
 * tensor -- `in` with `pads_before[d]` zeros in front of dim d, extents `padded_shape`, dense row-major -- is never
 * written; out[i0, i1, ..] is its element view_offset + sum(i_k * view_strides[k]), read from `in` when it lies in
 * the interior and zero otherwise.  One view stride per dim of `out`; 4-byte element types. */
int fluidml_hip_pad_view_copy(const fl_tensor *in, const int64_t *pads_before, const int64_t *padded_shape, int32_t n_dims, int64_t view_offset, const int64_t *view_strides, const fl_tensor *out, void *stream);
/* GatherConstantIndexScalarKernel (reference gather.cpp:100-139). */
int fluidml_hip_gather_constant_index_scalar(const fl_tensor *in, const fl_tensor *out, int64_t axis, int64_t index, uint32_t flags, void *stream);
/* GatherConstantIndicesTensorKernel: data is the runtime input, `indices` a
 * constant int64 tensor (reference gather.cpp:149-186, 24-86). */
int fluidml_hip_gather_constant_indices_tensor(const fl_tensor *in, const fl_tensor *indices, const fl_tensor *out, int64_t axis, void *stream);
/* GatherConstantDataTensorKernel: `data` is a constant float32 table, the
 * runtime input holds int64 indices, axis 0 (reference gather.cpp:195-272). */
int fluidml_hip_gather_constant_data_tensor(const fl_tensor *indices, const fl_tensor *data, const fl_tensor *out, void *stream);
/* GatherConstantDataTensorKernel -> AddCommonKernel as one launch: out = data[indices] + add0, add0 broadcast
 * to out (reference gather.cpp:224-262, add.cpp:75-137; the one-addend form of the fused kernel below). */
int fluidml_hip_gather_constant_data_tensor_add(const fl_tensor *indices, const fl_tensor *data, const fl_tensor *add0, const fl_tensor *out, void *stream);
/* GatherConstantDataTensorAddTensorLhsAddTensorLhsKernel: data[ids] + add0 + add1
 * (reference gather_add_add.cpp:25-163). */
int fluidml_hip_gather_constant_data_tensor_add_tensor_lhs_add_tensor_lhs(const fl_tensor *indices, const fl_tensor *data, const fl_tensor *add0, const fl_tensor *add1, const fl_tensor *out, void *stream);
/* CumSumKernel: integer inclusive forward scan (reference cum_sum.cpp:53-87). */
int fluidml_hip_cum_sum(const fl_tensor *in, const fl_tensor *out, int64_t axis, void *stream);

/* ------------------------------------------------------------------------- */
/* a.2 Row-reduction kernels (HBM bound).                                     */

/* SoftmaxKernel along `axis` (>= 0) (reference softmax.cpp:22-139).  The
 * reference makes six passes through a scratch of shape[axis->1]; here the
 * row is reduced in registers/LDS and `scratch` is not touched. */
int fluidml_hip_softmax(const fl_tensor *in, const fl_tensor *out, void *scratch, size_t scratch_bytes, int64_t axis, void *stream);
/* LayerNormalizationConstantScaleBiasKernel: biased variance over the single
 * `axis`; scale/bias broadcast from the trailing dims (reference
 * layer_normalization.cpp:33-220).  With FL_REF_LN_STALE_SCRATCH the row sum
 * starts from the float the scratch holds for that row. */
int fluidml_hip_layer_normalization_constant_scale_bias(const fl_tensor *in, const fl_tensor *scale, const fl_tensor *bias, const fl_tensor *out, void *scratch, size_t scratch_bytes, int64_t axis, double epsilon, uint32_t flags, void *stream);
/* ReduceMeanKernel, keepdims=1 only (reference reduce_mean.cpp:16-98). */
int fluidml_hip_reduce_mean(const fl_tensor *in, const fl_tensor *out, const int64_t *axes, int32_t n_axes, void *stream);
/* MaxPoolWithoutPaddingKernel: trailing `n` dims pooled (reference maxpool.cpp:17-82). */
int fluidml_hip_max_pool_without_padding(const fl_tensor *in, const fl_tensor *out, const int64_t *kernel_shape, const int64_t *strides, int32_t n, void *stream);
/* AveragePoolWithoutPaddingKernel (reference averagepool.cpp:19-87). */
int fluidml_hip_average_pool_without_padding(const fl_tensor *in, const fl_tensor *out, const int64_t *kernel_shape, const int64_t *strides, int32_t n, void *stream);

/* ------------------------------------------------------------------------- */
/* a.1 Contraction kernels (MFMA bound).                                      */

/* MatMulKernel: NumPy batch-broadcast matmul, fp32 MFMA
 * (reference matmul.cpp:28-59, utils.cpp:64-147). */
int fluidml_hip_matmul(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream);
/* fluidml_hip_matmul for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It
 * has no counterpart in the reference.  Same arguments, same kernels and the
 * same result bit for bit as fluidml_hip_matmul, but a launch that splits K
 * over several workgroups keeps its partial tiles and arrival counters in a
 * fixed device array inside the library (FL_NO_ALLOC_SCRATCH_BYTES of partial
 * tiles plus 8 KiB of counters per GPU, held until the process ends) instead
 * of the stream's workspace, and the call allocates nothing.  A problem whose
 * split needs more than the array holds (tiles x splits partial 32x32 tiles of
 * 4 KiB each: 96 tiles x 4 splits fit, 160 tiles x 4 splits do not) is refused with
 * FL_ERR_STATIC_SCRATCH and nothing is launched.  All calls on one GPU share
 * the array: calls that overlap in time on one GPU (two streams, two threads)
 * race; calls on one stream are ordered and safe. */
#define FL_NO_ALLOC_SCRATCH_BYTES (2u << 20)
int fluidml_hip_matmul_no_alloc(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream);
/* Same contraction with operands rounded to bf16 (nearest even) and fp32
 * accumulation on v_mfma_f32_32x32x8_bf16 (opt-in; no counterpart in the
 * reference, error is reported separately). */
int fluidml_hip_matmul_bf16(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *out, void *stream);
/* GemmConstantBiasKernel (kernel name "GemmConstantWeightsBiasKernel"):
 * rank-2, bias rank 1 or 2 (reference gemm.cpp:39-182). */
int fluidml_hip_gemm_constant_weights_bias(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out, double alpha, double beta, int32_t trans_a, int32_t trans_b, uint32_t flags, void *stream);
/* ConvWithoutPaddingKernel: NCHW-logical, N-d spatial, group==1 or depthwise
 * (reference conv.cpp:27-201, 214-218). bias may be NULL. `strides` and
 * `dilations` have rank-2 entries. */
int fluidml_hip_conv_without_padding(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out, const int64_t *strides, const int64_t *dilations, int64_t group, uint32_t flags, void *stream);
/* ConvWithPaddingKernel (reference conv.cpp:230-280). `pads` has 2*(rank-2)
 * entries, begins then ends.  The reference materialises the zero-padded
 * input in `scratch`; here padding is applied on the fly and scratch is
 * untouched. */
int fluidml_hip_conv_with_padding(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out, void *scratch, size_t scratch_bytes, const int64_t *pads, const int64_t *strides, const int64_t *dilations, int64_t group, uint32_t flags, void *stream);

/* ------------------------------------------------------------------------- */
/* Launch-level fusions.  Each computes exactly what the named chain of        */
/* kernels above computes, operation for operation, without writing the        */
/* chain's intermediate tensors; the launcher uses them where an intermediate  */
/* has one reader (the reference fuses at graph level instead, e.g.            */
/* add_div_erf_add_mul_mul.cpp, and has no launch-level counterpart).          */

/* MatMulKernel -> AddCommonKernel with a rank-1 bias over the last dim
 * (reference matmul.cpp:28-59 + add.cpp:75-137). */
int fluidml_hip_matmul_add(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out, void *stream);
/* MatMulKernel [-> AddCommonKernel(rank-1 bias)] -> elementwise chain on the
 * result, e.g. the erf-GELU chain Div, Erf, Add, Mul(x), Mul of
 * add_div_erf_add_mul_mul.cpp:29-132.  `bias` and `chain` may be NULL. */
int fluidml_hip_matmul_chain(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out, const fl_ew_program *chain, uint32_t flags, void *stream);
/* The same followed by one or two AddCommonKernel with tensors of the output's shape and strides (a residual
 * connection, or GPT-NeoX's parallel residual x + attention + mlp): out = (chain(lhs . rhs + bias) + addend) + addend2,
 * each sum rounded like the separate kernels' (reference matmul.cpp:28-59, add.cpp:75-137).  `addend2` may be NULL.
 * `rhs` must be unit-stride along its last dim, otherwise FL_ERR_UNSUPPORTED.  FL_CONTRACT_BF16 is honoured for dense
 * row-major operands with 16-byte aligned rows; other operands keep the launch in fp32. */
int fluidml_hip_matmul_chain_add(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out, const fl_ew_program *chain, const fl_tensor *addend, const fl_tensor *addend2, uint32_t flags, void *stream);
/* The same, followed by Reshape / Transpose steps that only re-address the
 * result (reference reshape.cpp:18-64, transpose.cpp:19-48): `out` carries the
 * contraction's logical shape [..., M, N] with the element strides each of
 * those dims has inside the final buffer.  If the reshape split N into
 * (N / n_inner, n_inner) and the transpose moved the two apart, column n is
 * stored at (n / n_inner) * stride_outer + (n % n_inner) * out->strides[last];
 * n_inner == 0 means plain strides. */
int fluidml_hip_matmul_chain_view(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out, int64_t n_inner, int64_t stride_outer, const fl_ew_program *chain, uint32_t flags, void *stream);
/* `count` (1..4) such launches that share `lhs`, every extent, the strides of
 * `rhs`, `n_inner` and `chain`, as ONE launch (the query / key / value
 * projections of an attention block): rhs[i], bias[i] (all NULL or none),
 * out[i] and stride_outer[i] belong to member i.  No batch dims. */
int fluidml_hip_matmul_chain_group(int32_t count, const fl_tensor *lhs, const fl_tensor *const *rhs, const fl_tensor *const *bias, const fl_tensor *const *out, int64_t n_inner, const int64_t *stride_outer, const fl_ew_program *chain, uint32_t flags, void *stream);
/* A LayerNormalization over the last axis that is kept out of memory between the contraction that produces its
 * input and the contractions that consume its output (reference layer_normalization.cpp:33-220 between
 * matmul.cpp:28-59 launches, e.g. the two post-attention / post-FFN normalisations of a transformer layer).  The
 * tensor t that would be normalised is stored as it is, together with partial row statistics: for row r and every
 * run j of 32 consecutive columns, stats[(r * parts + j) * 2 + 0] = mean and [.. + 1] = sum of squared deviations
 * of that run (parts = ceil(width / 32); Chan's pairwise update combines them without cancellation).  A consumer
 * then works on LayerNorm(t) = (t - mean_r) * rstd_r * scale + shift without it ever being written:
 *   deferred == FL_NORM_LHS: `lhs` of the call is t.  Because the normalisation is affine per row, the product is
 *     rstd_r * (t . (diag(scale) rhs) - mean_r * col_sum) + (shift . rhs + bias): the caller passes diag(scale) rhs
 *     as `rhs`, col_sum[n] = sum_k scale[k] rhs[k][n] per member as `col_sum[i]`, and shift . rhs + bias as `bias[i]`.
 *   deferred == FL_NORM_ADDEND: `addend` of the call is t; (t - mean_r) * rstd_r * scale[n] + shift[n] is added
 *     after the chain, where a plain addend would be.
 * `stats_out` (may be given with or without a deferred operand): the call leaves the partial statistics of its own
 * output rows there, ceil(N / 32) pairs per row, for the next consumer.  Single batch element only. */
enum fl_norm_deferred { FL_NORM_NONE = 0, FL_NORM_LHS = 1, FL_NORM_ADDEND = 2 };
typedef struct fl_norm_fusion {
  int32_t deferred;       /* enum fl_norm_deferred */
  int32_t width;          /* extent of the normalised axis of t */
  double epsilon;
  const float *stats;     /* partial statistics of t's rows (device memory), NULL if deferred == FL_NORM_NONE */
  const fl_tensor *scale; /* FL_NORM_ADDEND: rank-1 [N] */
  const fl_tensor *shift; /* FL_NORM_ADDEND: rank-1 [N] */
  float *stats_out;       /* NULL: none */
  const fl_tensor *addend2; /* NULL: none; a second tensor with the strides of out[0], added (plain) after `addend` */
} fl_norm_fusion;
/* fluidml_hip_matmul_chain_group (count 1..4; count == 1 is a single chain) with such a normalisation folded in.
 * `col_sum[i]`: rank-1 [N] per member, FL_NORM_LHS only (else NULL).  `addend`: a tensor with the strides of out[0]
 * added after the chain (plain, or t of FL_NORM_ADDEND); count == 1 and n_inner == 0 only.  FL_CONTRACT_BF16 rounds
 * the two operands of the contraction (with FL_NORM_LHS: the un-normalised left operand and the pre-scaled weights);
 * statistics, the epilogue's correction and the addends stay fp32.  The tile configuration bits of `flags` apply
 * (FL_TILE_128x128_STAGED: deferred rows of at most 512 elements). */
int fluidml_hip_matmul_chain_group_norm(int32_t count, const fl_tensor *lhs, const fl_tensor *const *rhs, const fl_tensor *const *bias, const fl_tensor *const *col_sum, const fl_tensor *const *out, int64_t n_inner, const int64_t *stride_outer, const fl_ew_program *chain, const fl_tensor *addend, const fl_norm_fusion *norm, uint32_t flags, void *stream);
/* GemmConstantWeightsBiasKernel -> elementwise chain (reference gemm.cpp:39-182); `flags` = fl_contract_flags. */
int fluidml_hip_gemm_chain(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *bias, const fl_tensor *out, double alpha, double beta, int32_t trans_a, int32_t trans_b, const fl_ew_program *chain, uint32_t flags, void *stream);
/* Conv{With,Without}PaddingKernel -> elementwise chain (reference conv.cpp:27-280);
 * `pads` may be NULL.  ONNX semantics only (no literal-reference flags); `flags` = fl_contract_flags. */
int fluidml_hip_conv_chain(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out, const int64_t *pads, const int64_t *strides, const int64_t *dilations, int64_t group, const fl_ew_program *chain, uint32_t flags, void *stream);
/* [MulCommonKernel(x, scale per channel) ->] Conv{With,Without}PaddingKernel -> elementwise chain [-> AddCommonKernel
 * with a tensor of the output's shape] as ONE launch (reference mul.cpp, conv.cpp:27-280, add.cpp:75-137: the
 * projection of an inverted-residual block behind its squeeze-and-excitation gate, with the skip connection).
 * Only for a 1x1 convolution with unit stride, no padding and group 1 whose pixels are one strided run in `in`
 * and `out` (it runs as a plain contraction; fp32 whatever `flags` say).  `channel_scale` ([1, C, 1, ..], NULL:
 * none) multiplies the input, each product rounded as the separate kernel rounds it; one image only.  `addend`
 * (NULL: none) has the shape and strides of `out`; with FL_CONTRACT_ADDEND_IS_FACTOR in `flags` the value is
 * multiplied by it instead (MulCommonKernel behind the convolution; `out` and `addend` may then both be a
 * transposed view, which is how a Transpose between the two is absorbed).  Anything else: FL_ERR_UNSUPPORTED,
 * nothing launched. */
int fluidml_hip_conv_chain_scale_add(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out, const int64_t *pads, const int64_t *strides, const int64_t *dilations, int64_t group, const fl_ew_program *chain, const fl_tensor *channel_scale, const fl_tensor *addend, uint32_t flags, void *stream);
/* Conv{With,Without}PaddingKernel -> elementwise chain -> ReduceMeanKernel over the spatial dims (keepdims) as ONE call
 * with two results (reference conv.cpp:27-280, reduce_mean.cpp: the depthwise convolution of an inverted-residual
 * block and the squeeze of its squeeze-and-excitation gate): `out` as for fluidml_hip_conv_chain, `mean_out`
 * [N, F, 1, ..] its mean over the spatial dims.  One launch for a depthwise 3x3 or 5x5 convolution with stride 1 or 2
 * whose padded input plane fits LDS (a workgroup per plane); otherwise the convolution, then the reduction. */
int fluidml_hip_conv_chain_mean(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out, const int64_t *pads, const int64_t *strides, const int64_t *dilations, int64_t group, const fl_ew_program *chain, const fl_tensor *mean_out, uint32_t flags, void *stream);
/* SoftmaxKernel over K <= 16 logits [B, K, 1] -> MatMulKernel [B, M, K] x [B, K, 1] as ONE launch:
 * out[b, m, 0] = sum_k a[b, m, k] * softmax_k(logits[b, :, 0]) (reference softmax.cpp, matmul.cpp:28-59; the
 * per-position kernel of a span-based dynamic convolution).  `out` is [B, M, 1] with the element strides
 * these dims have inside the final buffer (a following Reshape is free), or [B / I, I, M, 1] where the batches lie
 * in the final buffer as I at one stride under another (heads inside a part of a concatenated tensor).
 * K > 16: FL_ERR_UNSUPPORTED. */
int fluidml_hip_softmax_matvec(const fl_tensor *a, const fl_tensor *logits, const fl_tensor *out, void *stream);
/* Two pointwise convolutions on tensors of one pixel ([N, C, 1, ..]), each followed by an elementwise chain, as
 * ONE launch: the squeeze-and-excitation pair Conv -> activation -> Conv -> activation behind a global pooling
 * (reference conv.cpp:27-218 twice; both must have kernel size 1 and group 1, biases and chains may be NULL).
 * At most 4096 input channels and 512 channels in between, else FL_ERR_UNSUPPORTED and nothing is launched. */
int fluidml_hip_pointwise_conv_pair(const fl_tensor *in, const fl_tensor *weights1, const fl_tensor *bias1, const fl_ew_program *chain1, const fl_tensor *weights2, const fl_tensor *bias2, const fl_ew_program *chain2, const fl_tensor *out, void *stream);
/* A chain of elementwise kernels on one float32 tensor as one launch:
 * out = chain(in), same shape, any two layouts. */
int fluidml_hip_elementwise_chain(const fl_tensor *in, const fl_tensor *out, const fl_ew_program *chain, void *stream);
/* MulCommonKernel -> AddCommonKernel: out = a * b + c (product rounded, then the sum, like the two kernels);
 * a, b and c broadcast to out.  (reference mul.cpp:70-132, add.cpp:75-137) */
int fluidml_hip_mul_add(const fl_tensor *a, const fl_tensor *b, const fl_tensor *c, const fl_tensor *out, void *stream);
/* AddCommonKernel -> AddCommonKernel (two residual sums): out = (a + b) + c, rounded like the two kernels;
 * a, b and c broadcast to out.  (reference add.cpp:75-137) */
int fluidml_hip_add_add(const fl_tensor *a, const fl_tensor *b, const fl_tensor *c, const fl_tensor *out, void *stream);
/* The rotary position embedding of the exported GPT-NeoX graphs as one launch: Slice x[.., :R] and x[.., R:],
 * Slice the two halves of the first, NegKernel, Concat2Kernel (-second half, first half), MulCommonKernel with
 * the sine table, MulCommonKernel of x[.., :R] with the cosine table, AddCommonKernel, Concat2Kernel with
 * x[.., R:] (reference slice.cpp:17-55, neg.cpp:17-40, concat.cpp:18-68, mul.cpp:70-132, add.cpp:75-137).
 * With h = R / 2 and rot = concat(-x[.., h:R], x[.., :h]):
 *   out[.., d] = x[.., d] * cos[.., d] + rot[.., d] * sin[.., d]   for d < R = rotary_dims (even),
 *   out[.., d] = x[.., d]                                          beyond,
 * both products rounded before the sum, like the separate kernels (bit-identical to them).  cos and sin have R
 * values along the last axis; their leading dims broadcast to x's.  x and out: same shape, any strides. */
int fluidml_hip_rotary(const fl_tensor *x, const fl_tensor *cos_table, const fl_tensor *sin_table, const fl_tensor *out, int64_t rotary_dims, void *stream);
/* The same for two tensors against the same tables in ONE launch (the queries and the keys of an attention layer):
 * out0 = rotary(x0), out1 = rotary(x1); each pair (x, out) has one shape, the two pairs may differ. */
int fluidml_hip_rotary_pair(const fl_tensor *x0, const fl_tensor *out0, const fl_tensor *x1, const fl_tensor *out1, const fl_tensor *cos_table, const fl_tensor *sin_table, int64_t rotary_dims, void *stream);
/* DivConstantRhsKernel -> AddCommonKernel(mask, broadcast) -> SoftmaxKernel:
 * out = softmax(in / div + mask, axis)
 * (reference div.cpp:24-56 + add.cpp:75-137 + softmax.cpp:22-139). */
int fluidml_hip_div_add_softmax(const fl_tensor *in, double div, const fl_tensor *mask, const fl_tensor *out, int64_t axis, void *stream);
/* MatMulKernel -> DivConstantRhs | MulConstant -> [AddCommon(mask)] ->
 * [WhereConstantCondConstantScalarY] -> SoftmaxKernel(last axis) -> MatMulKernel:
 *   out = softmax(where(keep_cond, (q.kt) / scale (or * scale) + add_mask, fill)) . v
 * q [..., Sq, D], kt [..., D, Skv], v [..., Skv, D], out [..., Sq, D], equal
 * batch dims, any strides (a transposed or head-split view costs nothing);
 * add_mask (float32) and keep_cond (bool) broadcast to [..., Sq, Skv] and may
 * be NULL.  D <= 64 and Skv <= 256, otherwise FL_ERR_UNSUPPORTED (nothing
 * launched).  (reference matmul.cpp:28-59, div.cpp:24-56, add.cpp:75-137,
 * where.cpp:17-150, softmax.cpp:22-139) */
int fluidml_hip_attention(const fl_tensor *q, const fl_tensor *kt, const fl_tensor *v, const fl_tensor *out, double scale, int32_t scale_is_divisor, const fl_tensor *add_mask, const fl_tensor *keep_cond, double fill, void *stream);
/* GatherConstantDataTensorKernel whose result feeds a LayerNormalization that is not run (fl_norm_fusion): out =
 * data[indices] as fluidml_hip_gather_constant_data_tensor, and stats_out (device memory, 2 * ceil(len / 32) floats
 * per looked-up row) receives the partial row statistics of `out` in the layout of fl_norm_fusion.stats.  data
 * [rows, len], everything dense row-major, otherwise FL_ERR_UNSUPPORTED.  (reference gather.cpp:195-272,
 * layer_normalization.cpp:33-220) */
int fluidml_hip_gather_constant_data_tensor_stats(const fl_tensor *indices, const fl_tensor *data, const fl_tensor *out, float *stats_out, void *stream);
/* GatherConstantDataTensorKernel [x2] -> AddCommonKernel [-> AddCommonKernel] ->
 * LayerNormalizationConstantScaleBiasKernel over the last dim (the embedding
 * block of a BERT-style encoder) as one launch:
 *   out = LayerNorm((data0[indices0] + x) + third),
 *   x = second[indices1] when indices1 is given (`second` is then a table
 *   [rows1, len]), otherwise the tensor `second` itself.
 * data0 [rows0, len]; indices int64 of out's leading dims; out [..., len];
 * `second` (as a tensor) and `third` (may be NULL) have out's trailing dims
 * with nothing but ones in front (they repeat along the leading dims);
 * scale and bias hold len values.  Everything dense row-major and
 * len <= FL_GATHER_LAYER_NORM_MAX_LEN, otherwise FL_ERR_UNSUPPORTED and
 * nothing is launched.  The sums round as the separate kernels' do.
 * (reference gather.cpp:195-272, add.cpp:75-137, layer_normalization.cpp:33-220) */
#define FL_GATHER_LAYER_NORM_MAX_LEN 2048
int fluidml_hip_gather_add_layer_normalization(const fl_tensor *indices0, const fl_tensor *data0, const fl_tensor *indices1, const fl_tensor *second, const fl_tensor *third, const fl_tensor *scale, const fl_tensor *bias, const fl_tensor *out, double epsilon, void *stream);
/* AddCommonKernel -> LayerNormalizationConstantScaleBiasKernel:
 * out = LayerNorm(lhs + rhs) (reference add.cpp:75-137 +
 * layer_normalization.cpp:33-220, ONNX semantics). */
int fluidml_hip_add_layer_normalization(const fl_tensor *lhs, const fl_tensor *rhs, const fl_tensor *scale, const fl_tensor *bias, const fl_tensor *out, int64_t axis, double epsilon, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* FLUIDML_HIP_H_ */
