// Softmax along one axis in a single launch (HBM-bound: one read, one write).
//
// inner == 1 (rows of `channels` contiguous floats): one wavefront per row,
// max and sum by shuffle reduction, the row kept in registers when it fits;
// rows of at most 64 channels share a wavefront.
// inner  > 1 (channel stride = inner): one thread per (outer, inner) column,
// walking the channels; neighbouring threads read neighbouring addresses.
#include "mc_common.h"
#include "mchip/kernels.h"

#include <cfloat>

namespace mchip {
namespace {

constexpr int kRowRegs = 16;  // up to 64*16 = 1024 channels held in registers

__global__ __launch_bounds__(256) void softmax_rows_kernel(const float* __restrict__ x,
                                                           float* __restrict__ y, long rows,
                                                           int C) {
  const long row = blockIdx.x * 4L + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const float* __restrict__ xr = x + row * C;
  float* __restrict__ yr = y + row * C;
  float v[kRowRegs];
  float m = -FLT_MAX;
  if (C <= 64 * kRowRegs) {
#pragma unroll
    for (int i = 0; i < kRowRegs; ++i) {
      const int c = lane + 64 * i;
      v[i] = c < C ? xr[c] : -FLT_MAX;
      m = fmaxf(m, v[i]);
    }
  } else {
    for (int c = lane; c < C; c += 64) m = fmaxf(m, xr[c]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  float s = 0.f;
  if (C <= 64 * kRowRegs) {
#pragma unroll
    for (int i = 0; i < kRowRegs; ++i) {
      const int c = lane + 64 * i;
      v[i] = c < C ? expf(v[i] - m) : 0.f;
      s += v[i];
    }
  } else {
    for (int c = lane; c < C; c += 64) s += expf(xr[c] - m);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
  if (C <= 64 * kRowRegs) {
#pragma unroll
    for (int i = 0; i < kRowRegs; ++i) {
      const int c = lane + 64 * i;
      if (c < C) yr[c] = v[i] / s;
    }
  } else {
    for (int c = lane; c < C; c += 64) yr[c] = expf(xr[c] - m) / s;
  }
}

// Rows of at most G channels (G a power of two): G lanes per row, 64 / G rows
// per wavefront, one register per lane.  Lanes past the last row or channel
// take part in the shuffles with neutral values.
template <int G>
__global__ __launch_bounds__(256) void softmax_rows_small_kernel(const float* __restrict__ x,
                                                                 float* __restrict__ y, long rows,
                                                                 int C) {
  const long t = blockIdx.x * 256L + threadIdx.x;
  const long row = t / G;
  const int c = static_cast<int>(t % G);
  const bool on = row < rows && c < C;
  const float v = on ? x[row * C + c] : -FLT_MAX;
  float m = v;
#pragma unroll
  for (int o = G / 2; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  const float e = on ? expf(v - m) : 0.f;
  float s = e;
#pragma unroll
  for (int o = G / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
  if (on) y[row * C + c] = e / s;
}

template <int G>
void launch_softmax_rows_small(const float* x, float* y, long rows, int C, hipStream_t st) {
  const long blocks = ceil_div(rows * G, 256L);
  softmax_rows_small_kernel<G><<<static_cast<unsigned>(blocks), 256, 0, st>>>(x, y, rows, C);
}

__global__ __launch_bounds__(256) void softmax_cols_kernel(const float* __restrict__ x,
                                                           float* __restrict__ y, long columns,
                                                           int C, int inner) {
  for (long i = blockIdx.x * 256L + threadIdx.x; i < columns; i += gridDim.x * 256L) {
    const long o = i / inner, k = i - o * inner;
    const float* __restrict__ xc = x + o * C * inner + k;
    float* __restrict__ yc = y + o * C * inner + k;
    float m = xc[0];
    for (int c = 1; c < C; ++c) m = fmaxf(m, xc[(long)c * inner]);
    float s = 0.f;
    for (int c = 0; c < C; ++c) {
      const float e = expf(xc[(long)c * inner] - m);
      yc[(long)c * inner] = e;
      s += e;
    }
    for (int c = 0; c < C; ++c) yc[(long)c * inner] = yc[(long)c * inner] / s;
  }
}

}  // namespace
}  // namespace mchip

using namespace mchip;

extern "C" int mcSoftmax(const float* bottom, float* top, int outer, int channels, int inner,
                         void* stream) {
  MC_REQUIRE(bottom && top, "mcSoftmax: null argument");
  MC_REQUIRE(outer >= 0 && channels > 0 && inner > 0, "mcSoftmax: bad extents");
  if (outer == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (inner == 1 && channels <= 64) {
    if (channels <= 4) launch_softmax_rows_small<4>(bottom, top, outer, channels, st);
    else if (channels <= 8) launch_softmax_rows_small<8>(bottom, top, outer, channels, st);
    else if (channels <= 16) launch_softmax_rows_small<16>(bottom, top, outer, channels, st);
    else if (channels <= 32) launch_softmax_rows_small<32>(bottom, top, outer, channels, st);
    else launch_softmax_rows_small<64>(bottom, top, outer, channels, st);
  } else if (inner == 1) {
    softmax_rows_kernel<<<ceil_div(outer, 4), 256, 0, st>>>(bottom, top, outer, channels);
  } else {
    MC_REQUIRE(bottom != top, "mcSoftmax: in-place needs inner == 1");
    const long columns = (long)outer * inner;
    softmax_cols_kernel<<<ew_blocks(columns, 256), 256, 0, st>>>(bottom, top, columns, channels,
                                                                 inner);
  }
  MC_LAUNCH_CHECK();
  return 0;
}
