// Convolution kernels: NCHW-logical, N-d spatial (1..3 dims), group == 1 or
// depthwise, with or without padding.
// Reference: src/structure/kernel/kernel/conv.cpp:27-201 (loop nest n,f,c,o..,k..
// accumulating into the output), :214-218 (without padding), :230-280 (with
// padding: the zero-padded input is materialised in the node's scratch).
//
// Padding is applied on the fly (out-of-range taps contribute nothing), so the
// scratch bytes the memory plan reserves for ConvWithPadding stay untouched.
// Taps are accumulated in the reference's (c, k0, k1, ...) order.
#include "fl_common.h"

namespace fl {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxSpatial = 3;

struct ConvArgs {
  // canonical order of the output's (n, f, o...) index space; operand 0 = out offset, operand 1 = the logical
  // linear index (de-linearised back to (n, f, o...) in the kernel)
  NestArgs<2> out_nest;
  int32_t rank;          // 2 + n_spatial
  int32_t n_spatial;
  int32_t out_shape[2 + kMaxSpatial];
  int32_t in_shape[2 + kMaxSpatial];
  int32_t in_strides[2 + kMaxSpatial];
  int32_t w_strides[2 + kMaxSpatial];
  int32_t k_shape[kMaxSpatial];
  int32_t pad[kMaxSpatial];
  int32_t stride[kMaxSpatial];
  int32_t dilation[kMaxSpatial];
  int32_t channels;      // input channels per output channel (C for group==1, 1 for depthwise)
  int32_t depthwise;
  int32_t bias_stride;   // element stride of bias; 0 with bias_fixed
  int32_t bias_fixed;    // FL_REF_CONV_BIAS_INDEX1: every element gets bias[1]
  uint32_t n_out;
  fl_ew_program chain;   // elementwise chain applied after the bias (n == 0: none)
};

template <int NS>
__global__ __launch_bounds__(kBlock) void ConvDirect(ConvArgs p, float *__restrict__ out, const float *__restrict__ in,
                                                     const float *__restrict__ w, const float *__restrict__ bias) {
  const uint32_t item = blockIdx.x * kBlock + threadIdx.x;
  if (item >= p.n_out) return;
  // canonical index -> output offset and logical linear index
  int32_t both[2] = {0, 0};
  p.out_nest.AddOffsets(item, both);
  const int32_t ooff = both[0];
  int32_t lin = both[1];
  int32_t o[NS];
#pragma unroll
  for (int d = NS - 1; d >= 0; --d) {
    o[d] = lin % p.out_shape[2 + d];
    lin /= p.out_shape[2 + d];
  }
  const int32_t f = lin % p.out_shape[1];
  const int32_t n = lin / p.out_shape[1];

  const float *wf = w + f * p.w_strides[0];
  const float *inn = in + n * p.in_strides[0];
  int32_t base[NS];
#pragma unroll
  for (int d = 0; d < NS; ++d) base[d] = o[d] * p.stride[d] - p.pad[d];

  float acc = 0.0f;
  for (int32_t c = 0; c < p.channels; ++c) {
    const float *inc = inn + (p.depthwise ? f : c) * p.in_strides[1];
    const float *wc = wf + c * p.w_strides[1];
    if constexpr (NS == 1) {
      for (int32_t k0 = 0; k0 < p.k_shape[0]; ++k0) {
        const int32_t i0 = base[0] + k0 * p.dilation[0];
        if (i0 >= 0 && i0 < p.in_shape[2]) acc += inc[i0 * p.in_strides[2]] * wc[k0 * p.w_strides[2]];
      }
    } else if constexpr (NS == 2) {
      for (int32_t k0 = 0; k0 < p.k_shape[0]; ++k0) {
        const int32_t i0 = base[0] + k0 * p.dilation[0];
        if (i0 < 0 || i0 >= p.in_shape[2]) continue;
        for (int32_t k1 = 0; k1 < p.k_shape[1]; ++k1) {
          const int32_t i1 = base[1] + k1 * p.dilation[1];
          if (i1 >= 0 && i1 < p.in_shape[3])
            acc += inc[i0 * p.in_strides[2] + i1 * p.in_strides[3]] * wc[k0 * p.w_strides[2] + k1 * p.w_strides[3]];
        }
      }
    } else {
      for (int32_t k0 = 0; k0 < p.k_shape[0]; ++k0) {
        const int32_t i0 = base[0] + k0 * p.dilation[0];
        if (i0 < 0 || i0 >= p.in_shape[2]) continue;
        for (int32_t k1 = 0; k1 < p.k_shape[1]; ++k1) {
          const int32_t i1 = base[1] + k1 * p.dilation[1];
          if (i1 < 0 || i1 >= p.in_shape[3]) continue;
          for (int32_t k2 = 0; k2 < p.k_shape[2]; ++k2) {
            const int32_t i2 = base[2] + k2 * p.dilation[2];
            if (i2 >= 0 && i2 < p.in_shape[4])
              acc += inc[i0 * p.in_strides[2] + i1 * p.in_strides[3] + i2 * p.in_strides[4]] *
                     wc[k0 * p.w_strides[2] + k1 * p.w_strides[3] + k2 * p.w_strides[4]];
          }
        }
      }
    }
  }
  if (bias != nullptr) acc += p.bias_fixed ? bias[p.bias_stride] : bias[f * p.bias_stride];
  if (p.chain.n != 0) acc = RunChain(p.chain, acc);
  out[ooff] = acc;
}

}  // namespace

// matmul.hip
int ConvImplicitGemm(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out,
                     const int64_t *pads, const int64_t *strides, const int64_t *dilations,
                     const fl_ew_program *chain, void *stream);

namespace {

int Conv(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out,
         const int64_t *pads, const int64_t *strides, const int64_t *dilations, int64_t group, uint32_t flags,
         void *stream, const fl_ew_program *chain = nullptr) {
  FL_CHECK(CheckChain(chain));
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(weights));
  FL_CHECK(CheckView(out));
  if (in->dtype != FL_FLOAT32 || weights->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  const int rank = out->rank;
  if (rank < 3 || rank > 2 + kMaxSpatial) return FL_ERR_RANK;
  if (in->rank != rank || weights->rank != rank) return FL_ERR_RANK;
  const int ns = rank - 2;
  const int64_t N = in->shape[0], C = in->shape[1], F = out->shape[1];
  if (out->shape[0] != N || weights->shape[0] != F) return FL_ERR_SHAPE;
  if (group <= 0) return FL_ERR_ATTR;
  const bool depthwise = group != 1;
  if (!depthwise) {
    if (weights->shape[1] != C) return FL_ERR_SHAPE;
  } else {
    // reference conv.cpp:103-149 handles group != 1 only as w[f, 0, k...] * in[n, f, o+k]
    if (weights->shape[1] != 1 || C != F || group != C) return FL_ERR_UNSUPPORTED;
  }
  ConvArgs p;
  std::memset(&p, 0, sizeof(p));
  p.rank = rank;
  p.n_spatial = ns;
  p.channels = depthwise ? 1 : static_cast<int32_t>(C);
  p.depthwise = depthwise ? 1 : 0;
  if (chain != nullptr) p.chain = *chain;
  const bool unit = (flags & FL_REF_CONV_UNIT_STRIDE) != 0;
  for (int i = 0; i < rank; ++i) {
    p.out_shape[i] = static_cast<int32_t>(out->shape[i]);
    p.in_shape[i] = static_cast<int32_t>(in->shape[i]);
    p.in_strides[i] = static_cast<int32_t>(in->strides[i]);
    p.w_strides[i] = static_cast<int32_t>(weights->strides[i]);
  }
  for (int d = 0; d < ns; ++d) {
    p.k_shape[d] = static_cast<int32_t>(weights->shape[2 + d]);
    p.pad[d] = pads ? static_cast<int32_t>(pads[d]) : 0;
    const int64_t pad_end = pads ? pads[d + ns] : 0;
    p.stride[d] = (unit || !strides) ? 1 : static_cast<int32_t>(strides[d]);
    p.dilation[d] = (unit || !dilations) ? 1 : static_cast<int32_t>(dilations[d]);
    if (p.pad[d] < 0 || pad_end < 0 || p.stride[d] <= 0 || p.dilation[d] <= 0) return FL_ERR_ATTR;
    // the last tap of the last output must lie inside the padded input
    const int64_t last = (out->shape[2 + d] - 1) * p.stride[d] + (p.k_shape[d] - 1) * p.dilation[d];
    if (last >= in->shape[2 + d] + p.pad[d] + pad_end) return FL_ERR_SHAPE;
  }
  const float *b = nullptr;
  if (bias != nullptr) {
    FL_CHECK(CheckView(bias));
    if (bias->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    if (bias->rank != 1 || bias->shape[0] != F) return FL_ERR_SHAPE;
    b = static_cast<const float *>(bias->base);
    p.bias_stride = static_cast<int32_t>(bias->strides[0]);
    if (flags & FL_REF_CONV_BIAS_INDEX1) {
      if (F < 2) return FL_ERR_SHAPE;
      p.bias_fixed = 1;
    }
  }
  // dense contractions go to the matrix cores; depthwise, 3-d and literal-reference modes stay here
  if (!depthwise && flags == 0 && ns <= 2) {
    const int rc = ConvImplicitGemm(in, weights, bias, out, pads, strides, dilations, chain, stream);
    if (rc != FL_ERR_UNSUPPORTED) return rc;
  }
  LoopNest nest;
  nest.rank = rank;
  nest.n_operands = 2;
  int64_t acc = 1;
  for (int i = rank - 1; i >= 0; --i) {
    nest.shape[i] = out->shape[i];
    nest.strides[0][i] = out->strides[i];
    nest.strides[1][i] = acc;
    acc *= out->shape[i];
  }
  nest.Canonicalise();
  p.out_nest = MakeNestArgs<2>(nest);
  p.n_out = static_cast<uint32_t>(Numel(out));
  const dim3 grid((p.n_out + kBlock - 1) / kBlock), block(kBlock);
  float *o = static_cast<float *>(out->base);
  const float *x = static_cast<const float *>(in->base);
  const float *w = static_cast<const float *>(weights->base);
  hipStream_t s = AsStream(stream);
  switch (ns) {
    case 1: FL_LAUNCH(ConvDirect<1>, grid, block, 0, s, p, o, x, w, b); break;
    case 2: FL_LAUNCH(ConvDirect<2>, grid, block, 0, s, p, o, x, w, b); break;
    case 3: FL_LAUNCH(ConvDirect<3>, grid, block, 0, s, p, o, x, w, b); break;
    default: return FL_ERR_RANK;
  }
  return LaunchStatus();
}

}  // namespace
}  // namespace fl

extern "C" {

int fluidml_hip_conv_without_padding(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias,
                                     const fl_tensor *out, const int64_t *strides, const int64_t *dilations,
                                     int64_t group, uint32_t flags, void *stream) {
  return fl::Conv(in, weights, bias, out, nullptr, strides, dilations, group, flags, stream);
}

int fluidml_hip_conv_with_padding(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias,
                                  const fl_tensor *out, void *scratch, size_t scratch_bytes, const int64_t *pads,
                                  const int64_t *strides, const int64_t *dilations, int64_t group, uint32_t flags,
                                  void *stream) {
  (void)scratch;
  (void)scratch_bytes;
  if (pads == nullptr) return FL_ERR_NULL;
  return fl::Conv(in, weights, bias, out, pads, strides, dilations, group, flags, stream);
}

int fluidml_hip_conv_chain(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out,
                           const int64_t *pads, const int64_t *strides, const int64_t *dilations, int64_t group,
                           const fl_ew_program *chain, void *stream) {
  return fl::Conv(in, weights, bias, out, pads, strides, dilations, group, 0, stream, chain);
}

}  // extern "C"
