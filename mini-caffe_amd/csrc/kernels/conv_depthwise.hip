// Direct depthwise convolution (group == input channels): each output channel
// reads one input channel through kh*kw taps, 2*kh*kw FLOP per 4-byte output, so
// the layer is bound by HBM, not by the matrix pipe, and gains nothing from the
// implicit-GEMM kernel (whose tiles would hold one useful row).  It replaces the
// reference's per-group im2col + sgemm for such layers
// (base_conv_layer.cpp:254-271 with group == channels) and corresponds to its
// ConvolutionDepthwise kernel (conv_dw_layer.cu:8-72): taps are accumulated in
// (kh, kw) order.
//
// One thread per output element, neighbouring threads along the output row, so
// loads and stores are coalesced and the kh*kw overlapping reads of neighbouring
// outputs are served by L1/L2.  A workgroup covers 256 consecutive outputs of the
// flattened [num*Cout][Ho*Wo] array; the per-channel filter is read with plain
// loads (same address across most of a wavefront).
#include "conv_internal.h"
#include "mc_common.h"
#include "mchip/kernels.h"

namespace mchip {
namespace {

// TRANS = false compiles only "none" and ReLU; the double-precision tanh / exp of
// the other activations would otherwise be part of every launch's inner loop.
template <bool TRANS>
__device__ __forceinline__ float dw_act(float v, int act, float slope) {
  if (!TRANS) return (act == MC_ACT_RELU && !(v > 0.f)) ? v * slope : v;
  switch (act) {
    case MC_ACT_RELU:
      return v > 0.f ? v : v * slope;
    case MC_ACT_TANH:
      return static_cast<float>(tanh(static_cast<double>(v)));
    case MC_ACT_SIGMOID:
      return static_cast<float>(1. / (1. + exp(-static_cast<double>(v))));
    default:
      return v;
  }
}

// KH/KW > 0: compile-time taps (fully unrolled); 0: run-time extents.
template <int KH, int KW, bool TRANS>
__global__ __launch_bounds__(256) void depthwise_kernel(const DepthwiseArgs a, long count) {
  const int kh_n = KH ? KH : a.kh, kw_n = KW ? KW : a.kw;
  const int plane = a.Ho * a.Wo;
  for (long i = blockIdx.x * 256L + threadIdx.x; i < count; i += gridDim.x * 256L) {
    const unsigned iu = static_cast<unsigned>(i);    // count < 2^31: 32-bit divisions
    const unsigned row = iu / static_cast<unsigned>(a.Wo);
    const int wo = static_cast<int>(iu - row * a.Wo);
    const unsigned nc = iu / static_cast<unsigned>(plane);  // n * Cout + oc
    const int ho = static_cast<int>(row - nc * a.Ho);
    const unsigned cout = static_cast<unsigned>(a.C * a.mult);
    const long n = nc / cout;
    const int oc = static_cast<int>(nc - static_cast<unsigned>(n) * cout);
    const int c = oc / a.mult;
    const float* __restrict__ xp = a.x + (n * a.C + c) * a.H * a.W;
    const float* __restrict__ wp = a.w + static_cast<long>(oc) * kh_n * kw_n;
    const int hi0 = ho * a.sh - a.ph, wi0 = wo * a.sw - a.pw;
    float acc = 0.f;
#pragma unroll
    for (int r = 0; r < kh_n; ++r) {
      const int hi = hi0 + r * a.dh;
      const bool row_ok = static_cast<unsigned>(hi) < static_cast<unsigned>(a.H);
#pragma unroll
      for (int s = 0; s < kw_n; ++s) {
        const int wi = wi0 + s * a.dw;
        const bool ok = row_ok && static_cast<unsigned>(wi) < static_cast<unsigned>(a.W);
        const float v = ok ? xp[hi * a.W + wi] : 0.f;
        acc += wp[r * kw_n + s] * v;
      }
    }
    if (a.scale) acc *= a.scale[oc];
    if (a.shift) acc += a.shift[oc];
    if (a.residual) acc += a.residual[i];
    a.y[i] = dw_act<TRANS>(acc, a.act, a.slope);
  }
}

// Undilated kernels with stride SH down the column: a thread makes R
// vertically neighbouring outputs (same column, rows R*q .. R*q+R-1) from
// (R-1)*SH + KH input rows, so overlapping taps are read once per thread instead of
// once per output and the index arithmetic is shared; neighbouring threads sit on
// neighbouring columns, so every load and store stays coalesced.
template <int KH, int KW, int SH, bool TRANS, int R>
__global__ __launch_bounds__(256) void depthwise_rows_kernel(const DepthwiseArgs a, long groups,
                                                         int ho_groups) {
  constexpr int L = (R - 1) * SH + KH;
  for (long gi = blockIdx.x * 256L + threadIdx.x; gi < groups; gi += gridDim.x * 256L) {
    const unsigned gu = static_cast<unsigned>(gi);   // groups < 2^31
    const unsigned row = gu / static_cast<unsigned>(a.Wo);        // (n*Cout + oc)*ho_groups + q
    const int wo = static_cast<int>(gu - row * a.Wo);
    const unsigned nc = row / static_cast<unsigned>(ho_groups);
    const int ho0 = static_cast<int>(row - nc * ho_groups) * R;
    const unsigned cout = static_cast<unsigned>(a.C * a.mult);
    const unsigned n = nc / cout;
    const int oc = static_cast<int>(nc - n * cout);
    const int c = oc / a.mult;
    const float* __restrict__ xp = a.x + (static_cast<long>(n) * a.C + c) * a.H * a.W;
    const float* __restrict__ wp = a.w + static_cast<long>(oc) * KH * KW;
    const int hi0 = ho0 * SH - a.ph, wi0 = wo * a.sw - a.pw;
    float wv[KH][KW];
#pragma unroll
    for (int r = 0; r < KH; ++r)
#pragma unroll
      for (int s = 0; s < KW; ++s) wv[r][s] = wp[r * KW + s];
    float acc[R];
#pragma unroll
    for (int o = 0; o < R; ++o) acc[o] = 0.f;
#pragma unroll
    for (int t = 0; t < L; ++t) {
      const int hi = hi0 + t;
      const bool row_ok = static_cast<unsigned>(hi) < static_cast<unsigned>(a.H);
      float v[KW];
#pragma unroll
      for (int s = 0; s < KW; ++s) {
        const int wi = wi0 + s;
        const bool ok = row_ok && static_cast<unsigned>(wi) < static_cast<unsigned>(a.W);
        v[s] = ok ? xp[hi * a.W + wi] : 0.f;
      }
      // input row t is tap row t - o*SH of output o
#pragma unroll
      for (int o = 0; o < R; ++o) {
        const int r = t - o * SH;
        if (r >= 0 && r < KH) {
#pragma unroll
          for (int s = 0; s < KW; ++s) acc[o] += wv[r][s] * v[s];
        }
      }
    }
    const float sc = a.scale ? a.scale[oc] : 1.f, sf = a.shift ? a.shift[oc] : 0.f;
#pragma unroll
    for (int o = 0; o < R; ++o) {
      if (ho0 + o >= a.Ho) break;
      const long out = (static_cast<long>(nc) * a.Ho + ho0 + o) * a.Wo + wo;
      float val = acc[o];
      if (a.scale) val *= sc;
      if (a.shift) val += sf;
      if (a.residual) val += a.residual[out];
      a.y[out] = dw_act<TRANS>(val, a.act, a.slope);
    }
  }
}

}  // namespace

int depthwise_forward(const DepthwiseArgs& a, hipStream_t stream) {
  const long count = static_cast<long>(a.num) * a.C * a.mult * a.Ho * a.Wo;
  if (count == 0) return 0;
  const bool trans = a.act == MC_ACT_TANH || a.act == MC_ACT_SIGMOID;
  if (a.kh == 3 && a.kw == 3 && a.dh == 1 && a.dw == 1 && (a.sh == 1 || a.sh == 2)) {
    // R output rows per thread: more rows share more of their input rows (R + 2 rows
    // read for R outputs at stride 1), as long as the map is tall enough to keep
    // every thread's rows inside it
    const int rows = a.Ho >= 96 ? 16 : (a.Ho >= (a.sh == 1 ? 16 : 32) ? 8 : 4);
    const int ho_groups = ceil_div(a.Ho, rows);
    const long groups = static_cast<long>(a.num) * a.C * a.mult * ho_groups * a.Wo;
    const unsigned gb = ew_blocks(groups, 256);
#define MC_DW_LAUNCH(SH, R)                                                                   \
  if (trans) depthwise_rows_kernel<3, 3, SH, true, R><<<gb, 256, 0, stream>>>(a, groups, ho_groups); \
  else depthwise_rows_kernel<3, 3, SH, false, R><<<gb, 256, 0, stream>>>(a, groups, ho_groups)
    if (a.sh == 1) {
      if (rows == 16) { MC_DW_LAUNCH(1, 16); }
      else if (rows == 8) { MC_DW_LAUNCH(1, 8); }
      else { MC_DW_LAUNCH(1, 4); }
    } else {
      if (rows == 16) { MC_DW_LAUNCH(2, 16); }
      else if (rows == 8) { MC_DW_LAUNCH(2, 8); }
      else { MC_DW_LAUNCH(2, 4); }
    }
#undef MC_DW_LAUNCH
    MC_LAUNCH_CHECK();
    return 0;
  }
  const unsigned blocks = ew_blocks(count, 256);
  if (a.kh == 3 && a.kw == 3) {
    if (trans) depthwise_kernel<3, 3, true><<<blocks, 256, 0, stream>>>(a, count);
    else depthwise_kernel<3, 3, false><<<blocks, 256, 0, stream>>>(a, count);
  } else if (a.kh == 5 && a.kw == 5) {
    if (trans) depthwise_kernel<5, 5, true><<<blocks, 256, 0, stream>>>(a, count);
    else depthwise_kernel<5, 5, false><<<blocks, 256, 0, stream>>>(a, count);
  } else {
    if (trans) depthwise_kernel<0, 0, true><<<blocks, 256, 0, stream>>>(a, count);
    else depthwise_kernel<0, 0, false><<<blocks, 256, 0, stream>>>(a, count);
  }
  MC_LAUNCH_CHECK();
  return 0;
}

}  // namespace mchip
