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
  FastDiv out_div[2 + kMaxSpatial];  // division by out_shape[i]
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

// KH, KW: the window of the first two spatial dims when known at compile time (0 = read from the arguments): the tap
// loops then unroll and their loads are issued together instead of one round trip per tap.  Same order of the sums.
template <int NS, int KH = 0, int KW = 0>
__global__ __launch_bounds__(kBlock) void ConvDirect(ConvArgs p, float *__restrict__ out, const float *__restrict__ in,
                                                     const float *__restrict__ w, const float *__restrict__ bias) {
  const uint32_t item = blockIdx.x * kBlock + threadIdx.x;
  if (item >= p.n_out) return;
  // canonical index -> output offset and logical linear index
  int32_t both[2] = {0, 0};
  p.out_nest.AddOffsets(item, both);
  const int32_t ooff = both[0];
  uint32_t lin = static_cast<uint32_t>(both[1]);
  int32_t o[NS];
#pragma unroll
  for (int d = NS - 1; d >= 0; --d) {
    uint32_t q, r;
    p.out_div[2 + d].DivMod(lin, q, r);
    o[d] = static_cast<int32_t>(r);
    lin = q;
  }
  uint32_t n_u, f_u;
  p.out_div[1].DivMod(lin, n_u, f_u);
  const int32_t f = static_cast<int32_t>(f_u), n = static_cast<int32_t>(n_u);

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
      const int32_t kh = KH > 0 ? KH : p.k_shape[0];
#pragma unroll
      for (int32_t k0 = 0; k0 < kh; ++k0) {
        const int32_t i0 = base[0] + k0 * p.dilation[0];
        if (i0 >= 0 && i0 < p.in_shape[2]) acc += inc[i0 * p.in_strides[2]] * wc[k0 * p.w_strides[2]];
      }
    } else if constexpr (NS == 2) {
      const int32_t kh = KH > 0 ? KH : p.k_shape[0], kw = KW > 0 ? KW : p.k_shape[1];
#pragma unroll
      for (int32_t k0 = 0; k0 < kh; ++k0) {
        const int32_t i0 = base[0] + k0 * p.dilation[0];
        if (i0 < 0 || i0 >= p.in_shape[2]) continue;
#pragma unroll
        for (int32_t k1 = 0; k1 < kw; ++k1) {
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

// ---- depthwise 2-d convolution, one workgroup per channel plane ----------------------------------------------
// The kernel above gives every output element its own thread, which then walks its K x K window through global
// memory.  For a depthwise convolution whose zero-padded input plane fits LDS a workgroup stages the plane of one
// (image, channel) once and its threads compute that plane's outputs from there; taps are added in the same
// (kh, kw) order.  Owning a whole plane, the workgroup can also deliver the mean of its outputs -- what a
// ReduceMean over the spatial dims behind the convolution (a squeeze-and-excitation block) would compute.
struct PlaneArgs {
  int32_t H, W, OH, OW, stride, pad_h, pad_w, rows, pitch;  // rows x pitch floats are staged
  int32_t sXn, sXc, sXh, sXw, sOn, sOc, sOh, sOw, sWc, sWh, sWw;
  const float *bias;
  int32_t sB;
  float *mean;  // optional: [image, channel] -> mean of the plane's outputs
  int32_t sMn, sMc;
  float count;
  FastDiv div_ow, div_pitch;
  fl_ew_program chain;
};

template <int K>
__global__ __launch_bounds__(kBlock) void ConvDepthwisePlaneKernel(PlaneArgs p, float *__restrict__ out,
                                                                   const float *__restrict__ in,
                                                                   const float *__restrict__ w) {
  extern __shared__ __align__(16) float plane[];
  __shared__ float partial[kBlock / kWave];
  const int32_t c = blockIdx.x, n = blockIdx.y;
  const int tid = threadIdx.x;
  float wv[K * K];
#pragma unroll
  for (int t = 0; t < K * K; ++t) wv[t] = w[c * p.sWc + (t / K) * p.sWh + (t % K) * p.sWw];
  const float bias = p.bias != nullptr ? p.bias[c * p.sB] : 0.0f;
  const float *src = in + static_cast<int64_t>(n) * p.sXn + static_cast<int64_t>(c) * p.sXc;
  const uint32_t n_stage = static_cast<uint32_t>(p.rows * p.pitch);
  for (uint32_t i = tid; i < n_stage; i += kBlock) {
    uint32_t r, cc;
    p.div_pitch.DivMod(i, r, cc);
    const int32_t ih = static_cast<int32_t>(r) - p.pad_h, iw = static_cast<int32_t>(cc) - p.pad_w;
    const bool inside = static_cast<uint32_t>(ih) < static_cast<uint32_t>(p.H) && static_cast<uint32_t>(iw) < static_cast<uint32_t>(p.W);
    plane[i] = inside ? src[ih * p.sXh + iw * p.sXw] : 0.0f;
  }
  __syncthreads();
  float *dst = out + static_cast<int64_t>(n) * p.sOn + static_cast<int64_t>(c) * p.sOc;
  const uint32_t n_out = static_cast<uint32_t>(p.OH * p.OW);
  float sum = 0.0f;
  for (uint32_t o = tid; o < n_out; o += kBlock) {
    uint32_t oh, ow;
    p.div_ow.DivMod(o, oh, ow);
    const float *win = plane + static_cast<int32_t>(oh) * p.stride * p.pitch + static_cast<int32_t>(ow) * p.stride;
    float acc = 0.0f;
#pragma unroll
    for (int kh = 0; kh < K; ++kh)
#pragma unroll
      for (int kw = 0; kw < K; ++kw) acc += win[kh * p.pitch + kw] * wv[kh * K + kw];
    if (p.bias != nullptr) acc += bias;
    if (p.chain.n != 0) acc = RunChain(p.chain, acc);
    dst[static_cast<int32_t>(oh) * p.sOh + static_cast<int32_t>(ow) * p.sOw] = acc;
    sum += acc;
  }
  if (p.mean != nullptr) {
    sum = BlockReduce<kBlock / kWave>(sum, SumOp{}, partial);
    if (tid == 0) p.mean[static_cast<int64_t>(n) * p.sMn + static_cast<int64_t>(c) * p.sMc] = sum / p.count;
  }
}

// FL_ERR_UNSUPPORTED (nothing launched) when the convolution does not fit: the caller goes on to the kernel above.
// `mean_out` (may be null): [N, C, 1, 1].
int ConvDepthwisePlane(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out,
                       const int64_t *pads, const int64_t *strides, const int64_t *dilations, const fl_ew_program *chain,
                       const fl_tensor *mean_out, void *stream) {
  // (read at every call: a test can switch the path inside one process)
  const char *plane_switch = std::getenv("FLUIDML_CONV_PLANE");
  const bool on = plane_switch == nullptr || std::strtol(plane_switch, nullptr, 10) != 0;
  if (!on || out->rank != 4) return FL_ERR_UNSUPPORTED;
  const int64_t N = in->shape[0], C = in->shape[1], H = in->shape[2], W = in->shape[3];
  const int64_t OH = out->shape[2], OW = out->shape[3], K = weights->shape[2];
  if (weights->shape[3] != K || (K != 3 && K != 5)) return FL_ERR_UNSUPPORTED;
  const int64_t st = strides ? strides[0] : 1;
  if ((strides && strides[1] != st) || st < 1 || st > 2) return FL_ERR_UNSUPPORTED;
  if (dilations && (dilations[0] != 1 || dilations[1] != 1)) return FL_ERR_UNSUPPORTED;
  const int64_t ph = pads ? pads[0] : 0, pw = pads ? pads[1] : 0;
  if (ph < 0 || pw < 0 || OH <= 0 || OW <= 0) return FL_ERR_UNSUPPORTED;
  const int64_t rows = (OH - 1) * st + K, pitch = (OW - 1) * st + K;
  // the plane has to be small and there have to be enough planes to fill the chip
  // (measured on EfficientNet-B0 at batch 1: planes of 14 x 14 to 30 x 30 with 240 to 1152 channels 4.3-6.5 against
  // 4.9-7.6 us for the kernel above plus 4 us for the separate mean; 144 planes of 60 x 60 11 against 8 us, 96 planes
  // of 114 x 114 29 against 7 us: too few workgroups, each staging too much)
  if (rows * pitch > 48 * 48 || N * C < 192 || N > 65535) return FL_ERR_UNSUPPORTED;
  if (Numel(in) > 0x7fffffff || Numel(out) > 0x7fffffff) return FL_ERR_UNSUPPORTED;
  PlaneArgs p;
  std::memset(&p, 0, sizeof(p));
  p.H = static_cast<int32_t>(H), p.W = static_cast<int32_t>(W), p.OH = static_cast<int32_t>(OH), p.OW = static_cast<int32_t>(OW);
  p.stride = static_cast<int32_t>(st), p.pad_h = static_cast<int32_t>(ph), p.pad_w = static_cast<int32_t>(pw);
  p.rows = static_cast<int32_t>(rows), p.pitch = static_cast<int32_t>(pitch);
  p.sXn = static_cast<int32_t>(in->strides[0]), p.sXc = static_cast<int32_t>(in->strides[1]);
  p.sXh = static_cast<int32_t>(in->strides[2]), p.sXw = static_cast<int32_t>(in->strides[3]);
  p.sOn = static_cast<int32_t>(out->strides[0]), p.sOc = static_cast<int32_t>(out->strides[1]);
  p.sOh = static_cast<int32_t>(out->strides[2]), p.sOw = static_cast<int32_t>(out->strides[3]);
  p.sWc = static_cast<int32_t>(weights->strides[0]), p.sWh = static_cast<int32_t>(weights->strides[2]);
  p.sWw = static_cast<int32_t>(weights->strides[3]);
  if (bias != nullptr) {
    p.bias = static_cast<const float *>(bias->base);
    p.sB = static_cast<int32_t>(bias->strides[0]);
  }
  if (mean_out != nullptr) {
    p.mean = static_cast<float *>(mean_out->base);
    p.sMn = static_cast<int32_t>(mean_out->strides[0]);
    p.sMc = static_cast<int32_t>(mean_out->strides[1]);
  }
  p.count = static_cast<float>(OH * OW);
  p.div_ow = FastDiv(static_cast<uint32_t>(OW));
  p.div_pitch = FastDiv(static_cast<uint32_t>(pitch));
  if (chain != nullptr) p.chain = *chain;
  const dim3 grid(static_cast<uint32_t>(C), static_cast<uint32_t>(N));
  const size_t lds = static_cast<size_t>(rows * pitch) * sizeof(float);
  float *o = static_cast<float *>(out->base);
  const float *x = static_cast<const float *>(in->base), *wp = static_cast<const float *>(weights->base);
  if (K == 3) FL_LAUNCH(ConvDepthwisePlaneKernel<3>, grid, dim3(kBlock), lds, AsStream(stream), p, o, x, wp);
  else FL_LAUNCH(ConvDepthwisePlaneKernel<5>, grid, dim3(kBlock), lds, AsStream(stream), p, o, x, wp);
  return LaunchStatus();
}

}  // namespace

// matmul.hip
int ConvImplicitGemm(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out,
                     const int64_t *pads, const int64_t *strides, const int64_t *dilations,
                     const fl_ew_program *chain, bool bf16, void *stream, const ConvExtras *extras);

int ConvHalo3x3(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out,
                const int64_t *pads, const int64_t *strides, const int64_t *dilations, const fl_ew_program *chain,
                void *stream, bool bf16);  // conv_halo.hip

namespace {

int Conv(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out,
         const int64_t *pads, const int64_t *strides, const int64_t *dilations, int64_t group, uint32_t flags,
         void *stream, const fl_ew_program *chain = nullptr, const ConvExtras *extras = nullptr) {
  const fl_tensor *mean_out = extras != nullptr ? extras->mean_out : nullptr;
  if (mean_out != nullptr) {
    FL_CHECK(CheckView(mean_out));
    if (mean_out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
    if (mean_out->rank != out->rank || mean_out->shape[0] != out->shape[0] || mean_out->shape[1] != out->shape[1]) return FL_ERR_SHAPE;
    for (int i = 2; i < mean_out->rank; ++i) {
      if (mean_out->shape[i] != 1) return FL_ERR_SHAPE;
    }
    if (extras->channel_scale != nullptr || extras->addend != nullptr) return FL_ERR_UNSUPPORTED;
  }
  if (extras != nullptr && extras->channel_scale == nullptr && extras->addend == nullptr) extras = nullptr;
  FL_CHECK(CheckChain(chain));
  FL_CHECK(CheckView(in));
  FL_CHECK(CheckView(weights));
  FL_CHECK(CheckView(out));
  if (in->dtype != FL_FLOAT32 || weights->dtype != FL_FLOAT32 || out->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  // the upper half of `flags` carries fl_contract_flags, the lower half fl_ref_flags
  const bool bf16 = ((flags >> FL_CONTRACT_SHIFT) & FL_CONTRACT_BF16) != 0;
  flags &= (1u << FL_CONTRACT_SHIFT) - 1;
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
    p.out_div[i] = FastDiv(static_cast<uint32_t>(out->shape[i]));
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
  if (depthwise && flags == 0 && ns == 2) {
    const int rc = ConvDepthwisePlane(in, weights, bias, out, pads, strides, dilations, chain, mean_out, stream);
    if (rc != FL_ERR_UNSUPPORTED) return rc;
  }
  if (mean_out != nullptr) {
    // no kernel delivers the mean with the result here: the convolution, then the reduction
    ConvExtras none;
    FL_CHECK(Conv(in, weights, bias, out, pads, strides, dilations, group, flags | (bf16 ? FL_CONTRACT_BF16 << FL_CONTRACT_SHIFT : 0u),
                  stream, chain, &none));
    int64_t axes[kMaxSpatial];
    for (int d = 0; d < ns; ++d) axes[d] = 2 + d;
    return fluidml_hip_reduce_mean(out, mean_out, axes, ns, stream);
  }
  if (extras != nullptr) {
    // the extra operands exist in the matrix-core path only
    if (depthwise || flags != 0 || ns > 2) return FL_ERR_UNSUPPORTED;
    return ConvImplicitGemm(in, weights, bias, out, pads, strides, dilations, chain, bf16, stream, extras);
  }
  if (!depthwise && flags == 0 && ns == 2) {
    // 3x3, unit stride: the input patch is staged once per workgroup instead of gathered tap by tap (with bf16
    // operands where they are allowed and the channels come in chunks of 16, else fp32)
    const int rc = ConvHalo3x3(in, weights, bias, out, pads, strides, dilations, chain, stream, bf16);
    if (rc != FL_ERR_UNSUPPORTED) return rc;
  }
  if (!depthwise && flags == 0 && ns <= 2) {
    const int rc = ConvImplicitGemm(in, weights, bias, out, pads, strides, dilations, chain, bf16, stream, nullptr);
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
    case 1:
      if (p.k_shape[0] == 9) {
        FL_LAUNCH((ConvDirect<1, 9>), grid, block, 0, s, p, o, x, w, b);
      } else if (p.k_shape[0] == 3) {
        FL_LAUNCH((ConvDirect<1, 3>), grid, block, 0, s, p, o, x, w, b);
      } else {
        FL_LAUNCH(ConvDirect<1>, grid, block, 0, s, p, o, x, w, b);
      }
      break;
    case 2:
      if (p.k_shape[0] == 3 && p.k_shape[1] == 3) {
        FL_LAUNCH((ConvDirect<2, 3, 3>), grid, block, 0, s, p, o, x, w, b);
      } else if (p.k_shape[0] == 5 && p.k_shape[1] == 5) {
        FL_LAUNCH((ConvDirect<2, 5, 5>), grid, block, 0, s, p, o, x, w, b);
      } else {
        FL_LAUNCH(ConvDirect<2>, grid, block, 0, s, p, o, x, w, b);
      }
      break;
    case 3: FL_LAUNCH(ConvDirect<3>, grid, block, 0, s, p, o, x, w, b); break;
    default: return FL_ERR_RANK;
  }
  return LaunchStatus();
}

// ---- two pointwise convolutions on one pixel (squeeze-and-excitation) ---------------------------------------
// hidden[s] = chain1(sum_c w1[s][c] * in[c] + b1[s]);  out[f] = chain2(sum_s w2[f][s] * hidden[s] + b2[f]).
// A workgroup of 16 waves owns 1024 outputs f of one image and recomputes the whole hidden vector (a few thousand
// multiply-adds).  Everything here is a chain of dependent round trips to memory, so each phase issues all its
// loads before it uses any: the input goes to LDS; wave w takes hidden channels w, w + 16, .. ROWS at a time, its
// lanes holding up to QUADS 128-bit pieces of each weight row (wave64 shuffle sum); then one lane per output walks
// its weight row (up to 48 values of it requested ahead) against the hidden vector in LDS.
constexpr int kPairBlock = 1024;
constexpr int kPairMaxChannels = 4096, kPairMaxHidden = 512;

struct ConvPairArgs {
  int32_t channels, hidden, outputs;
  int32_t in_n, in_c, out_n, out_f;  // element strides
  int32_t w1_s, w1_c, w2_f, w2_s;
  int32_t b1_stride, b2_stride;      // 0: no bias (the pointer is null)
  int32_t vec1, vec2;                // rows of w1 / w2 can be read 16 bytes at a time
  fl_ew_program chain1, chain2;
};

struct alignas(16) PairQuad {
  float v[4];
};

template <int QUADS, int ROWS>
__global__ __launch_bounds__(kPairBlock) void ConvPairKernel(ConvPairArgs p, float *__restrict__ out,
                                                             const float *__restrict__ in,
                                                             const float *__restrict__ w1, const float *__restrict__ b1,
                                                             const float *__restrict__ w2, const float *__restrict__ b2) {
  __shared__ __align__(16) float x[kPairMaxChannels];
  __shared__ __align__(16) float hidden[kPairMaxHidden];
  constexpr int kWaves = kPairBlock / kWave;
  // 128-bit pieces of an output's weight row requested before the hidden vector is known (fewer where the rows of
  // the first phase leave fewer registers)
  constexpr int kAhead = ROWS * QUADS > 8 ? 8 : 12;
  const int image = blockIdx.y;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int f = blockIdx.x * kPairBlock + threadIdx.x;
  const bool live = f < p.outputs;
  const float *row2 = w2 + static_cast<int64_t>(live ? f : 0) * p.w2_f;
  const int n_quads = p.channels / 4, hidden_quads = p.hidden / 4;
  // Every round trip to memory counts here (the weights are cold: nothing has read them since the last
  // inference), so the loads of both phases are requested as early as their registers allow: a wave's ROWS rows
  // of the first weight matrix and the first four pieces of the output's row before the input is staged, the
  // next eight pieces as soon as the first phase's products are done.
  PairQuad a[ROWS][QUADS], wq[kAhead];  // (wq[0..3] double as the sixteen scalars of a row that cannot be read 128 bits at a time)
  auto load_rows = [&](int s0) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int s = s0 + r * kWaves < p.hidden ? s0 + r * kWaves : s0;
      const PairQuad *row = reinterpret_cast<const PairQuad *>(w1 + static_cast<int64_t>(s) * p.w1_s);
#pragma unroll
      for (int k = 0; k < QUADS; ++k) {
        const int q = lane + k * kWave;
        a[r][k] = q < n_quads ? row[q] : PairQuad{{0, 0, 0, 0}};
      }
    }
  };
  auto load_quads = [&](int q0, int k0, int k1) {  // pieces q0 + k0 .. q0 + k1 - 1 into wq[k0 .. k1 - 1]
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
      if (k >= k0 && k < k1) wq[k] = q0 + k < hidden_quads ? reinterpret_cast<const PairQuad *>(row2)[q0 + k] : PairQuad{{0, 0, 0, 0}};
    }
  };
  auto load_scalars = [&](int s0) {
#pragma unroll
    for (int k = 0; k < 16; ++k) wq[k / 4].v[k % 4] = s0 + k < p.hidden ? row2[(s0 + k) * p.w2_s] : 0.0f;
  };
  if (p.vec1 && wave < p.hidden) load_rows(wave);
  if (live) {
    if (p.vec2) load_quads(0, 0, 4);
    else load_scalars(0);
  }
  // the biases too: a load issued only after the sums are known would be one more trip to memory each
  float bias_first[ROWS], bias_out = 0.0f;
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    bias_first[r] = b1 != nullptr && wave + r * kWaves < p.hidden ? b1[(wave + r * kWaves) * p.b1_stride] : 0.0f;
  }
  if (b2 != nullptr && live) bias_out = b2[f * p.b2_stride];
  const float *src = in + static_cast<int64_t>(image) * p.in_n;
  for (int c = threadIdx.x; c < p.channels; c += kPairBlock) x[c] = src[c * p.in_c];
  __syncthreads();
  if (p.vec1) {
    for (int s0 = wave; s0 < p.hidden; s0 += ROWS * kWaves) {
      if (s0 != wave) load_rows(s0);
      float acc[ROWS];
#pragma unroll
      for (int r = 0; r < ROWS; ++r) acc[r] = 0.0f;
#pragma unroll
      for (int k = 0; k < QUADS; ++k) {
        const int q = lane + k * kWave;
        if (q < n_quads) {
          const PairQuad xv = reinterpret_cast<const PairQuad *>(x)[q];
#pragma unroll
          for (int r = 0; r < ROWS; ++r)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[r] += a[r][k].v[e] * xv.v[e];
        }
      }
      if (s0 == wave && p.vec2 && live) load_quads(0, 4, kAhead);
#pragma unroll
      for (int r = 0; r < ROWS; ++r) acc[r] = WaveReduce(acc[r], SumOp{});
      if (lane == 0) {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
          const int s = s0 + r * kWaves;
          if (s < p.hidden) {
            float v = acc[r];
            if (b1 != nullptr) v += s0 == wave ? bias_first[r] : b1[s * p.b1_stride];
            hidden[s] = p.chain1.n != 0 ? RunChain(p.chain1, v) : v;
          }
        }
      }
    }
    if (wave >= p.hidden && p.vec2 && live) load_quads(0, 4, kAhead);  // waves without a row of the first phase
  } else {
    if (p.vec2 && live) load_quads(0, 4, kAhead);
    for (int s = wave; s < p.hidden; s += kWaves) {
      const float *row = w1 + static_cast<int64_t>(s) * p.w1_s;
      float acc = 0.0f;
#pragma unroll 8
      for (int c = lane; c < p.channels; c += kWave) acc += row[c * p.w1_c] * x[c];
      acc = WaveReduce(acc, SumOp{});
      if (lane == 0) {
        if (b1 != nullptr) acc += b1[s * p.b1_stride];
        hidden[s] = p.chain1.n != 0 ? RunChain(p.chain1, acc) : acc;
      }
    }
  }
  __syncthreads();
  if (!live) return;
  float acc = 0.0f;
  if (p.vec2) {
    for (int q0 = 0; q0 < hidden_quads; q0 += kAhead) {
      if (q0 != 0) load_quads(q0, 0, kAhead);
#pragma unroll
      for (int k = 0; k < kAhead; ++k) {
        if (q0 + k < hidden_quads) {
          const PairQuad h = reinterpret_cast<const PairQuad *>(hidden)[q0 + k];
#pragma unroll
          for (int e = 0; e < 4; ++e) acc += wq[k].v[e] * h.v[e];
        }
      }
    }
  } else {
    for (int s0 = 0; s0 < p.hidden; s0 += 16) {
      if (s0 != 0) load_scalars(s0);
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        if (s0 + k < p.hidden) acc += wq[k / 4].v[k % 4] * hidden[s0 + k];
      }
    }
  }
  acc += bias_out;
  if (p.chain2.n != 0) acc = RunChain(p.chain2, acc);
  out[static_cast<int64_t>(image) * p.out_n + static_cast<int64_t>(f) * p.out_f] = acc;
}

// One of the two convolutions above on its own, for the case where the weights are too many for one or two compute
// units to pull in reasonable time (1152 channels x 48 hidden values: 440 KB, 15 us in the kernel above): LANES lanes
// (64 or 16) share an output, walk its weight row 128 bits at a time and add their sums with shuffles, so that the rows
// spread over hundreds of waves; the hidden vector then travels through the stream's workspace between two launches.
template <int LANES>
__global__ __launch_bounds__(kBlock) void PointwiseOnePixelKernel(int32_t channels, int32_t outputs, int32_t in_n, int32_t in_c,
                                                                  int32_t out_n, int32_t out_f, int32_t w_f, int32_t w_c,
                                                                  int32_t b_stride, int32_t vec, fl_ew_program chain,
                                                                  float *__restrict__ out, const float *__restrict__ in,
                                                                  const float *__restrict__ w, const float *__restrict__ b) {
  constexpr int kRows = kBlock / LANES;
  const int image = blockIdx.y;
  const int f = blockIdx.x * kRows + threadIdx.x / LANES, lane = threadIdx.x % LANES;
  const bool live = f < outputs;
  const float *row = w + static_cast<int64_t>(live ? f : 0) * w_f;
  const float *x = in + static_cast<int64_t>(image) * in_n;
  float acc = 0.0f;
  if (vec) {
    for (int q = lane; q < channels / 4; q += LANES) {
      const PairQuad wv = reinterpret_cast<const PairQuad *>(row)[q], xv = reinterpret_cast<const PairQuad *>(x)[q];
#pragma unroll
      for (int e = 0; e < 4; ++e) acc += wv.v[e] * xv.v[e];
    }
  } else {
    for (int c = lane; c < channels; c += LANES) acc += row[c * w_c] * x[c * in_c];
  }
#pragma unroll
  for (int off = LANES / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, kWave);
  if (live && lane == 0) {
    if (b != nullptr) acc += b[f * b_stride];
    if (chain.n != 0) acc = RunChain(chain, acc);
    out[static_cast<int64_t>(image) * out_n + static_cast<int64_t>(f) * out_f] = acc;
  }
}

// [N, C, 1...] tensors: every dim from the third on has extent 1
inline bool OnePixel(const fl_tensor *t) {
  if (t->rank < 2) return false;
  for (int i = 2; i < t->rank; ++i) {
    if (t->shape[i] != 1) return false;
  }
  return true;
}

int ConvPair(const fl_tensor *in, const fl_tensor *w1, const fl_tensor *b1, const fl_ew_program *chain1,
             const fl_tensor *w2, const fl_tensor *b2, const fl_ew_program *chain2, const fl_tensor *out, void *stream) {
  if (!in || !w1 || !w2 || !out) return FL_ERR_NULL;
  const fl_tensor *all[6] = {in, w1, w2, out, b1, b2};
  for (const fl_tensor *t : all) {
    if (t == nullptr) continue;
    FL_CHECK(CheckView(t));
    if (t->dtype != FL_FLOAT32) return FL_ERR_DTYPE;
  }
  if (!OnePixel(in) || !OnePixel(w1) || !OnePixel(w2) || !OnePixel(out)) return FL_ERR_SHAPE;
  const int64_t n = in->shape[0], c = in->shape[1], s = w1->shape[0], f = w2->shape[0];
  if (w1->shape[1] != c || w2->shape[1] != s || out->shape[0] != n || out->shape[1] != f) return FL_ERR_SHAPE;
  if ((b1 && Numel(b1) != s) || (b2 && Numel(b2) != f)) return FL_ERR_SHAPE;
  if (c > kPairMaxChannels || s > kPairMaxHidden || n > 65535) return FL_ERR_UNSUPPORTED;
  if (n == 0 || f == 0) return FL_OK;
  auto last_stride = [](const fl_tensor *t) {  // element stride of a tensor with one non-unit dim
    for (int i = 0; i < t->rank; ++i) {
      if (t->shape[i] != 1) return static_cast<int32_t>(t->strides[i]);
    }
    return int32_t{1};
  };
  ConvPairArgs p;
  std::memset(&p, 0, sizeof(p));
  p.channels = static_cast<int32_t>(c);
  p.hidden = static_cast<int32_t>(s);
  p.outputs = static_cast<int32_t>(f);
  p.in_n = static_cast<int32_t>(in->strides[0]);
  p.in_c = static_cast<int32_t>(in->strides[1]);
  p.out_n = static_cast<int32_t>(out->strides[0]);
  p.out_f = static_cast<int32_t>(out->strides[1]);
  p.w1_s = static_cast<int32_t>(w1->strides[0]);
  p.w1_c = static_cast<int32_t>(w1->strides[1]);
  p.w2_f = static_cast<int32_t>(w2->strides[0]);
  p.w2_s = static_cast<int32_t>(w2->strides[1]);
  p.b1_stride = b1 ? last_stride(b1) : 0;
  p.b2_stride = b2 ? last_stride(b2) : 0;
  if (chain1 != nullptr) p.chain1 = *chain1;
  if (chain2 != nullptr) p.chain2 = *chain2;
  if (p.chain1.n > FL_EW_MAX_STEPS || p.chain2.n > FL_EW_MAX_STEPS) return FL_ERR_ATTR;
  p.vec1 = c % 4 == 0 && p.w1_c == 1 && p.w1_s % 4 == 0 && IsAligned(w1->base, 16) ? 1 : 0;
  p.vec2 = s % 4 == 0 && p.w2_s == 1 && p.w2_f % 4 == 0 && IsAligned(w2->base, 16) ? 1 : 0;
  // Many weights: two launches over many waves each, the hidden vector in the stream's workspace in between
  // (EfficientNet-B0's last blocks, 1152 x 48: 15 us in one launch).
  const char *split_switch = std::getenv("FLUIDML_PAIR_SPLIT_KB");
  const int64_t split_bytes = (split_switch != nullptr ? std::strtol(split_switch, nullptr, 10) : 64) * int64_t{1024};
  if ((c * s + s * f) * 4 >= split_bytes && n * s <= static_cast<int64_t>(kWorkspaceTiles * kWorkspaceTileFloats)) {
    if (StreamWorkspace *ws = GetStreamWorkspace(AsStream(stream))) {
      float *hidden = ws->partials;
      const int32_t hn = static_cast<int32_t>(s);
      const bool x_vec = p.vec1 && p.in_c == 1 && p.in_n % 4 == 0 && IsAligned(in->base, 16);
      const bool h_vec = p.vec2 && s % 4 == 0;
      const fl_ew_program none{};
      FL_LAUNCH(PointwiseOnePixelKernel<64>, dim3(static_cast<uint32_t>((s + 3) / 4), static_cast<uint32_t>(n)), dim3(kBlock), 0,
                AsStream(stream), p.channels, p.hidden, p.in_n, p.in_c, hn, 1, p.w1_s, p.w1_c, p.b1_stride, x_vec ? 1 : 0,
                chain1 ? *chain1 : none, hidden, static_cast<const float *>(in->base), static_cast<const float *>(w1->base),
                b1 ? static_cast<const float *>(b1->base) : nullptr);
      FL_LAUNCH(PointwiseOnePixelKernel<16>, dim3(static_cast<uint32_t>((f + 15) / 16), static_cast<uint32_t>(n)), dim3(kBlock), 0,
                AsStream(stream), p.hidden, p.outputs, hn, 1, p.out_n, p.out_f, p.w2_f, p.w2_s, p.b2_stride, h_vec ? 1 : 0,
                chain2 ? *chain2 : none, static_cast<float *>(out->base), hidden, static_cast<const float *>(w2->base),
                b2 ? static_cast<const float *>(b2->base) : nullptr);
      return LaunchStatus();
    }
  }
  const dim3 grid(static_cast<uint32_t>((f + kPairBlock - 1) / kPairBlock), static_cast<uint32_t>(n));
#define FL_CONV_PAIR(QUADS, ROWS)                                                                                  \
  FL_LAUNCH((ConvPairKernel<QUADS, ROWS>), grid, dim3(kPairBlock), 0, AsStream(stream), p, static_cast<float *>(out->base), \
            static_cast<const float *>(in->base), static_cast<const float *>(w1->base),                           \
            b1 ? static_cast<const float *>(b1->base) : nullptr, static_cast<const float *>(w2->base),            \
            b2 ? static_cast<const float *>(b2->base) : nullptr)
  if (c > 8 * 256) p.vec1 = 0;  // rows of more than 2048 values do not fit a wave's registers: strided loop
  // 128-bit pieces per lane and row, and rows of the first matrix per wave and trip (16 waves share them): all of
  // them in one trip while the registers last
  const int rows = s <= 16 ? 1 : s <= 32 ? 2 : 3;
  if (c <= 256) {
    if (rows == 1) FL_CONV_PAIR(1, 1);
    else if (rows == 2) FL_CONV_PAIR(1, 2);
    else FL_CONV_PAIR(1, 3);
  } else if (c <= 2 * 256) {
    if (rows == 1) FL_CONV_PAIR(2, 1);
    else if (rows == 2) FL_CONV_PAIR(2, 2);
    else FL_CONV_PAIR(2, 3);
  } else if (c <= 3 * 256) {
    if (rows == 1) FL_CONV_PAIR(3, 1);
    else if (rows == 2) FL_CONV_PAIR(3, 2);
    else FL_CONV_PAIR(3, 3);
  } else if (c <= 5 * 256) {  // (three rows of five pieces spill registers and were measured no faster)
    if (rows == 1) FL_CONV_PAIR(5, 1);
    else FL_CONV_PAIR(5, 2);
  } else {
    FL_CONV_PAIR(8, 1);
  }
#undef FL_CONV_PAIR
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
                           const fl_ew_program *chain, uint32_t flags, void *stream) {
  return fl::Conv(in, weights, bias, out, pads, strides, dilations, group, (flags & FL_CONTRACT_BF16) << FL_CONTRACT_SHIFT, stream,
                  chain);
}

int fluidml_hip_conv_chain_scale_add(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias,
                                     const fl_tensor *out, const int64_t *pads, const int64_t *strides,
                                     const int64_t *dilations, int64_t group, const fl_ew_program *chain,
                                     const fl_tensor *channel_scale, const fl_tensor *addend, uint32_t flags,
                                     void *stream) {
  fl::ConvExtras extras;
  extras.channel_scale = channel_scale;
  extras.addend = addend;
  extras.addend_is_factor = (flags & FL_CONTRACT_ADDEND_IS_FACTOR) != 0;
  if (extras.addend_is_factor && addend == nullptr) return FL_ERR_NULL;
  return fl::Conv(in, weights, bias, out, pads, strides, dilations, group, (flags & FL_CONTRACT_BF16) << FL_CONTRACT_SHIFT, stream,
                  chain, &extras);
}

int fluidml_hip_conv_chain_mean(const fl_tensor *in, const fl_tensor *weights, const fl_tensor *bias, const fl_tensor *out,
                                const int64_t *pads, const int64_t *strides, const int64_t *dilations, int64_t group,
                                const fl_ew_program *chain, const fl_tensor *mean_out, uint32_t flags, void *stream) {
  if (mean_out == nullptr) return FL_ERR_NULL;
  fl::ConvExtras extras;
  extras.mean_out = mean_out;
  return fl::Conv(in, weights, bias, out, pads, strides, dilations, group, (flags & FL_CONTRACT_BF16) << FL_CONTRACT_SHIFT, stream,
                  chain, &extras);
}

int fluidml_hip_pointwise_conv_pair(const fl_tensor *in, const fl_tensor *weights1, const fl_tensor *bias1,
                                    const fl_ew_program *chain1, const fl_tensor *weights2, const fl_tensor *bias2,
                                    const fl_ew_program *chain2, const fl_tensor *out, void *stream) {
  return fl::ConvPair(in, weights1, bias1, chain1, weights2, bias2, chain2, out, stream);
}

}  // extern "C"
