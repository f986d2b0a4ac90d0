// Max / average pooling (HBM-bound).
//
// Windowed pooling: one thread per output element, output width fastest, so a
// wavefront reads a contiguous span of each input row it touches.  Global
// pooling (window == image, one output per plane): one wavefront per plane with
// a shuffle reduction.
#include "mc_common.h"
#include "mchip/kernels.h"

#include <cfloat>
#include <cmath>
#include <cstdint>

namespace mchip {
namespace {

struct PoolArgs {
  const float* __restrict__ x;
  float* __restrict__ y;
  long total;  // planes*Ho*Wo
  int H, W, Ho, Wo;
  int kh, kw, sh, sw, ph, pw;
};

template <int METHOD>
__global__ __launch_bounds__(256) void pool_kernel(const PoolArgs a) {
  for (long i = blockIdx.x * 256L + threadIdx.x; i < a.total; i += gridDim.x * 256L) {
    const int ow = static_cast<int>(i % a.Wo);
    const long t = i / a.Wo;
    const int oh = static_cast<int>(t % a.Ho);
    const long plane = t / a.Ho;
    const float* __restrict__ xp = a.x + plane * a.H * a.W;
    int hs = oh * a.sh - a.ph, ws = ow * a.sw - a.pw;
    if (METHOD == MC_POOL_MAX) {
      const int he = min(hs + a.kh, a.H), we = min(ws + a.kw, a.W);
      hs = max(hs, 0);
      ws = max(ws, 0);
      float m = -FLT_MAX;
      for (int h = hs; h < he; ++h)
        for (int w = ws; w < we; ++w) m = fmaxf(m, xp[h * a.W + w]);
      a.y[i] = m;
    } else {
      int he = min(hs + a.kh, a.H + a.ph), we = min(ws + a.kw, a.W + a.pw);
      const int area = (he - hs) * (we - ws);
      hs = max(hs, 0);
      ws = max(ws, 0);
      he = min(he, a.H);
      we = min(we, a.W);
      float s = 0.f;
      for (int h = hs; h < he; ++h)
        for (int w = ws; w < we; ++w) s += xp[h * a.W + w];
      a.y[i] = s / static_cast<float>(area);
    }
  }
}

// Max pooling with a compile-time window and stride, padding 0 or more, for the
// shapes the model zoo uses (3x3/2 ResNet stem, 2x2/2 VGG, 3x3/1 SSD pool5): one
// thread makes two vertically adjacent outputs of a column, so the rows the two
// windows share are read once, all loads are issued before the first compare, and
// there is no loop-carried address arithmetic.  Neighbouring threads take
// neighbouring output columns.
template <int KH, int KW, int SH, int SW>
__global__ __launch_bounds__(256) void max_pool_fixed_kernel(const PoolArgs a, int row_pairs,
                                                             long count) {
  constexpr int ROWS = SH + KH;  // input rows under two vertically adjacent windows
  const long i = blockIdx.x * 256L + threadIdx.x;
  if (i >= count) return;
  const int ow = static_cast<int>(i % a.Wo);
  const long t = i / a.Wo;
  const int op = static_cast<int>(t % row_pairs);
  const long plane = t / row_pairs;
  const int oh = 2 * op;
  const float* __restrict__ xp = a.x + plane * a.H * a.W;
  const int h0 = oh * SH - a.ph, w0 = ow * SW - a.pw;
  float v[ROWS][KW];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int h = h0 + r;
    const bool hok = h >= 0 && h < a.H;
#pragma unroll
    for (int c = 0; c < KW; ++c) {
      const int w = w0 + c;
      v[r][c] = (hok && w >= 0 && w < a.W) ? xp[h * a.W + w] : -FLT_MAX;
    }
  }
  float m0 = -FLT_MAX, m1 = -FLT_MAX;
#pragma unroll
  for (int r = 0; r < KH; ++r)
#pragma unroll
    for (int c = 0; c < KW; ++c) {
      m0 = fmaxf(m0, v[r][c]);
      m1 = fmaxf(m1, v[r + SH][c]);
    }
  float* __restrict__ yp = a.y + (plane * a.Ho + oh) * a.Wo + ow;
  yp[0] = m0;
  if (oh + 1 < a.Ho) yp[a.Wo] = m1;
}

template <int KH, int KW, int SH, int SW>
void launch_max_pool_fixed(const PoolArgs& a, long planes, hipStream_t st) {
  const int row_pairs = (a.Ho + 1) / 2;
  const long count = planes * row_pairs * a.Wo;
  max_pool_fixed_kernel<KH, KW, SH, SW>
      <<<ceil_div(count, 256), 256, 0, st>>>(a, row_pairs, count);
}

// MAX 3x3 / stride 2 without padding on a width that is a multiple of 4 (the ResNet
// stem: 112 -> 56): one thread makes a 2 x 2 block of outputs from the 5 x 5 inputs under
// it, each input row as one aligned 16-byte load plus one more value, so neighbouring
// threads read neighbouring 16-byte pieces and every byte fetched is used; the block's
// two output rows leave as 8-byte stores when the output width is even.
__global__ __launch_bounds__(256) void max_pool_3x3s2_quad_kernel(const PoolArgs a, int row_pairs,
                                                                  int col_pairs, long count) {
  const long i = blockIdx.x * 256L + threadIdx.x;
  if (i >= count) return;
  const int cp = static_cast<int>(i % col_pairs);
  const long t = i / col_pairs;
  const int rp = static_cast<int>(t % row_pairs);
  const long plane = t / row_pairs;
  const float* __restrict__ xp = a.x + plane * a.H * a.W;
  const int h0 = 4 * rp, w0 = 4 * cp;
  const bool last_col = w0 + 4 < a.W;  // the fifth column exists
  float left[5], right[5];             // per input row: max of columns 0..2 and of columns 2..4
#pragma unroll
  for (int r = 0; r < 5; ++r) {
    left[r] = right[r] = -FLT_MAX;
    if (h0 + r < a.H) {
      const float* __restrict__ row = xp + (h0 + r) * a.W + w0;
      const float4 v = *reinterpret_cast<const float4*>(row);
      const float e = last_col ? row[4] : -FLT_MAX;
      left[r] = fmaxf(fmaxf(v.x, v.y), v.z);
      right[r] = fmaxf(fmaxf(v.z, v.w), e);
    }
  }
  const int oh = 2 * rp, ow = 2 * cp;
  const float t0 = fmaxf(fmaxf(left[0], left[1]), left[2]), t1 = fmaxf(fmaxf(right[0], right[1]), right[2]);
  const float b0 = fmaxf(fmaxf(left[2], left[3]), left[4]), b1 = fmaxf(fmaxf(right[2], right[3]), right[4]);
  float* __restrict__ yp = a.y + (plane * a.Ho + oh) * a.Wo + ow;
  const bool two_cols = ow + 1 < a.Wo, two_rows = oh + 1 < a.Ho;
  if (two_cols && (a.Wo & 1) == 0) {
    *reinterpret_cast<float2*>(yp) = make_float2(t0, t1);
    if (two_rows) *reinterpret_cast<float2*>(yp + a.Wo) = make_float2(b0, b1);
  } else {
    yp[0] = t0;
    if (two_cols) yp[1] = t1;
    if (two_rows) {
      yp[a.Wo] = b0;
      if (two_cols) yp[a.Wo + 1] = b1;
    }
  }
}

// G lanes per plane (a power of two up to the wavefront), 256 / G planes per
// workgroup: a 7x7 plane keeps 16 lanes busy for four loads each instead of 49
// lanes of a whole wavefront for one.
template <int METHOD, int G>
__global__ __launch_bounds__(256) void global_pool_kernel(const float* __restrict__ x,
                                                          float* __restrict__ y, long planes,
                                                          int hw) {
  const long plane = blockIdx.x * static_cast<long>(256 / G) + threadIdx.x / G;
  const int lane = threadIdx.x % G;
  float v = METHOD == MC_POOL_MAX ? -FLT_MAX : 0.f;
  if (plane < planes) {
    const float* __restrict__ xp = x + plane * hw;
    for (int i = lane; i < hw; i += G) {
      if (METHOD == MC_POOL_MAX) v = fmaxf(v, xp[i]);
      else v += xp[i];
    }
  }
#pragma unroll
  for (int o = G / 2; o > 0; o >>= 1) {
    const float u = __shfl_xor(v, o, 64);
    if (METHOD == MC_POOL_MAX) v = fmaxf(v, u);
    else v += u;
  }
  if (lane == 0 && plane < planes) y[plane] = METHOD == MC_POOL_MAX ? v : v / static_cast<float>(hw);
}

template <int METHOD>
void launch_global_pool(const float* x, float* y, long planes, int hw, hipStream_t st) {
  // about four values per lane, at least 8 lanes
  if (hw <= 32)
    global_pool_kernel<METHOD, 8><<<ceil_div(planes, 32), 256, 0, st>>>(x, y, planes, hw);
  else if (hw <= 64)
    global_pool_kernel<METHOD, 16><<<ceil_div(planes, 16), 256, 0, st>>>(x, y, planes, hw);
  else if (hw <= 128)
    global_pool_kernel<METHOD, 32><<<ceil_div(planes, 8), 256, 0, st>>>(x, y, planes, hw);
  else
    global_pool_kernel<METHOD, 64><<<ceil_div(planes, 4), 256, 0, st>>>(x, y, planes, hw);
}

}  // namespace
}  // namespace mchip

using namespace mchip;

extern "C" {

int mcPoolingOutputShape(int H, int W, int kh, int kw, int sh, int sw, int ph, int pw, int* Ho,
                         int* Wo) {
  MC_REQUIRE(kh > 0 && kw > 0, "Filter dimensions cannot be zero.");
  MC_REQUIRE(sh > 0 && sw > 0, "Stride dimensions cannot be zero.");
  MC_REQUIRE(ph >= 0 && pw >= 0 && ((ph == 0 && pw == 0) || (ph < kh && pw < kw)),
             "pad must be smaller than the kernel");
  int ho = static_cast<int>(std::ceil(static_cast<float>(H + 2 * ph - kh) / sh)) + 1;
  int wo = static_cast<int>(std::ceil(static_cast<float>(W + 2 * pw - kw) / sw)) + 1;
  if (ph || pw) {
    // The last window must start strictly inside the image, not in the padding.
    if ((ho - 1) * sh >= H + ph) --ho;
    if ((wo - 1) * sw >= W + pw) --wo;
  }
  MC_REQUIRE(ho > 0 && wo > 0, "mcPoolingOutputShape: empty output");
  if (Ho) *Ho = ho;
  if (Wo) *Wo = wo;
  return 0;
}

int mcPooling(int method, const float* bottom, float* top, int planes, int H, int W, int kh,
              int kw, int sh, int sw, int ph, int pw, void* stream) {
  MC_REQUIRE(bottom && top, "mcPooling: null argument");
  MC_REQUIRE(method == MC_POOL_MAX || method == MC_POOL_AVE, "Unknown pooling method.");
  MC_REQUIRE(planes >= 0 && H > 0 && W > 0, "mcPooling: bad extents");
  int Ho, Wo;
  if (mcPoolingOutputShape(H, W, kh, kw, sh, sw, ph, pw, &Ho, &Wo)) return -1;
  if (planes == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (Ho == 1 && Wo == 1 && kh >= H && kw >= W && ph == 0 && pw == 0) {
    if (method == MC_POOL_MAX) launch_global_pool<MC_POOL_MAX>(bottom, top, planes, H * W, st);
    else launch_global_pool<MC_POOL_AVE>(bottom, top, planes, H * W, st);
    MC_LAUNCH_CHECK();
    return 0;
  }
  PoolArgs a;
  a.x = bottom;
  a.y = top;
  a.total = (long)planes * Ho * Wo;
  a.H = H;
  a.W = W;
  a.Ho = Ho;
  a.Wo = Wo;
  a.kh = kh;
  a.kw = kw;
  a.sh = sh;
  a.sw = sw;
  a.ph = ph;
  a.pw = pw;
  if (method == MC_POOL_MAX && a.total < (1L << 31)) {
    // every window holds at least one element (the output shape guarantees it), so
    // the padding value never reaches the output
    bool done = true;
    if (kh == 3 && kw == 3 && sh == 2 && sw == 2 && ph == 0 && pw == 0 && W % 4 == 0 &&
        (reinterpret_cast<uintptr_t>(bottom) & 15u) == 0 && (reinterpret_cast<uintptr_t>(top) & 7u) == 0) {
      const int row_pairs = (Ho + 1) / 2, col_pairs = (Wo + 1) / 2;
      const long count = (long)planes * row_pairs * col_pairs;
      max_pool_3x3s2_quad_kernel<<<ceil_div(count, 256), 256, 0, st>>>(a, row_pairs, col_pairs, count);
    } else if (kh == 3 && kw == 3 && sh == 2 && sw == 2) launch_max_pool_fixed<3, 3, 2, 2>(a, planes, st);
    else if (kh == 2 && kw == 2 && sh == 2 && sw == 2) launch_max_pool_fixed<2, 2, 2, 2>(a, planes, st);
    else if (kh == 3 && kw == 3 && sh == 1 && sw == 1) launch_max_pool_fixed<3, 3, 1, 1>(a, planes, st);
    else done = false;
    if (done) {
      MC_LAUNCH_CHECK();
      return 0;
    }
  }
  const int blocks = ew_blocks(a.total, 256);
  if (method == MC_POOL_MAX) pool_kernel<MC_POOL_MAX><<<blocks, 256, 0, st>>>(a);
  else pool_kernel<MC_POOL_AVE><<<blocks, 256, 0, st>>>(a);
  MC_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
