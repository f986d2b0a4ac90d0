// L2 normalisation across channels (per pixel) or across the whole image.
#include "mc_common.h"
#include "mchip/kernels.h"

namespace mchip {
namespace {

// One thread per (image, pixel): neighbouring threads read neighbouring pixels
// of each channel plane, so every pass over the channels is coalesced.
__global__ __launch_bounds__(256) void normalize_pixel_kernel(
    const float* __restrict__ x, float* __restrict__ y, long pixels, int C, int spatial,
    int channel_shared, float eps, const float* __restrict__ scale) {
  for (long i = blockIdx.x * 256L + threadIdx.x; i < pixels; i += gridDim.x * 256L) {
    const long n = i / spatial, s = i - n * spatial;
    const float* __restrict__ xp = x + n * C * spatial + s;
    float* __restrict__ yp = y + n * C * spatial + s;
    float acc = eps;
    for (int c = 0; c < C; ++c) {
      const float v = xp[(long)c * spatial];
      acc += v * v;
    }
    const float norm = sqrtf(acc);
    for (int c = 0; c < C; ++c) {
      const float v = xp[(long)c * spatial] / norm;
      yp[(long)c * spatial] = v * (channel_shared ? scale[0] : scale[c]);
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
    const long pixels = (long)num * spatial;
    normalize_pixel_kernel<<<ew_blocks(pixels, 256), 256, 0, st>>>(
        bottom, top, pixels, channels, spatial, channel_shared, eps, scale);
  }
  MC_LAUNCH_CHECK();
  return 0;
}
