// L2 normalisation across channels (per pixel) or across the whole image.
#include "mc_common.h"
#include "mchip/kernels.h"

namespace mchip {
namespace {

// A workgroup takes 32 consecutive pixels of one image; its 8 groups of 32
// threads each sum every eighth channel, so a half-wave reads 128 contiguous
// bytes of a channel plane and a pixel's channels are covered by 8 threads
// instead of one serial walk.  The 8 partial sums are added in a fixed order.
// KEEP > 0: a thread's channels (at most KEEP of them, i.e. up to 8 * KEEP channels) stay
// in registers between the sum and the scaling, so the blob is read once.
constexpr int kNormPix = 32, kNormSlices = 8;
template <int KEEP>
__global__ __launch_bounds__(256) void normalize_pixel_kernel(
    const float* __restrict__ x, float* __restrict__ y, int C, int spatial, int tiles_per_image,
    int channel_shared, float eps, const float* __restrict__ scale) {
  __shared__ float part[kNormSlices][kNormPix];
  const int n = blockIdx.x / tiles_per_image;
  const int tile = blockIdx.x - n * tiles_per_image;
  const int px = threadIdx.x % kNormPix, sl = threadIdx.x / kNormPix;
  const int s = tile * kNormPix + px;
  const bool live = s < spatial;
  const float* __restrict__ xp = x + (long)n * C * spatial + s;
  float* __restrict__ yp = y + (long)n * C * spatial + s;
  float acc = 0.f;
  float kept[KEEP > 0 ? KEEP : 1];
  if (live) {
    if constexpr (KEEP > 0) {
      // all loads are independent: the whole column of this thread is in flight at once;
      // the squares are added in channel order, as the re-reading form below does
#pragma unroll
      for (int k = 0; k < KEEP; ++k) {
        const int c = sl + k * kNormSlices;
        kept[k] = c < C ? xp[(long)c * spatial] : 0.f;
      }
#pragma unroll
      for (int k = 0; k < KEEP; ++k) acc += kept[k] * kept[k];
    } else {
      // batches of 8 independent loads: the launch is small, so memory latency
      // has to be covered inside a thread
#pragma unroll 8
      for (int c = sl; c < C; c += kNormSlices) {
        const float v = xp[(long)c * spatial];
        acc += v * v;
      }
    }
  }
  part[sl][px] = acc;
  __syncthreads();
  float sum = eps;
#pragma unroll
  for (int k = 0; k < kNormSlices; ++k) sum += part[k][px];
  const float norm = sqrtf(sum);
  if (live) {
    if constexpr (KEEP > 0) {
#pragma unroll
      for (int k = 0; k < KEEP; ++k) {
        const int c = sl + k * kNormSlices;
        if (c < C) yp[(long)c * spatial] = (kept[k] / norm) * (channel_shared ? scale[0] : scale[c]);
      }
    } else {
#pragma unroll 8
      for (int c = sl; c < C; c += kNormSlices) {
        const float v = xp[(long)c * spatial] / norm;
        yp[(long)c * spatial] = v * (channel_shared ? scale[0] : scale[c]);
      }
    }
  }
}

// One workgroup per image.
__global__ __launch_bounds__(256) void normalize_image_kernel(
    const float* __restrict__ x, float* __restrict__ y, int C, int spatial, int channel_shared,
    float eps, const float* __restrict__ scale) {
  __shared__ float red[4];
  const long dim = (long)C * spatial;
  const float* __restrict__ xp = x + blockIdx.x * dim;
  float* __restrict__ yp = y + blockIdx.x * dim;
  float acc = 0.f;
  for (long i = threadIdx.x; i < dim; i += 256) acc += xp[i] * xp[i];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  const float norm = sqrtf(red[0] + red[1] + red[2] + red[3] + eps);
  const float inv = 1.0f / norm;
  for (long i = threadIdx.x; i < dim; i += 256) {
    const int c = static_cast<int>(i / spatial);
    yp[i] = (xp[i] * inv) * (channel_shared ? scale[0] : scale[c]);
  }
}

}  // namespace
}  // namespace mchip

using namespace mchip;

extern "C" int mcNormalize(const float* bottom, float* top, int num, int channels, int spatial,
                           int across_spatial, int channel_shared, float eps, const float* scale,
                           void* stream) {
  MC_REQUIRE(bottom && top && scale, "mcNormalize: null argument");
  MC_REQUIRE(num >= 0 && channels > 0 && spatial > 0, "mcNormalize: bad extents");
  if (num == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (across_spatial) {
    normalize_image_kernel<<<num, 256, 0, st>>>(bottom, top, channels, spatial, channel_shared,
                                                eps, scale);
  } else {
    const int tiles = ceil_div(spatial, kNormPix);
    MC_REQUIRE((long)num * tiles < (1L << 31), "mcNormalize: too many pixels");
    if (channels <= 16 * kNormSlices)
      normalize_pixel_kernel<16><<<num * tiles, 256, 0, st>>>(bottom, top, channels, spatial, tiles,
                                                             channel_shared, eps, scale);
    else if (channels <= 64 * kNormSlices)
      normalize_pixel_kernel<64><<<num * tiles, 256, 0, st>>>(bottom, top, channels, spatial, tiles,
                                                             channel_shared, eps, scale);
    else
      normalize_pixel_kernel<0><<<num * tiles, 256, 0, st>>>(bottom, top, channels, spatial, tiles,
                                                            channel_shared, eps, scale);
  }
  MC_LAUNCH_CHECK();
  return 0;
}
