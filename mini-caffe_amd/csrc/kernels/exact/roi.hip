// Region pooling over Proposal's rois: ROIPooling (max) and PSROIPooling
// (position-sensitive average).  One thread per output element, the same
// expressions and the same row-major accumulation order as the reference's CPU
// code (roi_pooling_layer.cpp:37-110, psroi_pooling_layer.cpp:45-122), compiled
// without contraction, so the results are the reference's bits.
//
// A roi whose batch index is outside [0, num) (the reference CHECK-fails on it
// on the CPU) yields zeros and raises *bad_roi_flag when the caller passes one.
#include "../mc_common.h"
#include "mchip/kernels.h"

#include <cfloat>

namespace mchip {
namespace {

struct RoiArgs {
  const float* bottom;
  const float* rois;
  float* top;
  int* bad_flag;
  int num, channels, height, width;
  int pooled_h, pooled_w;
  int group_size, output_dim;
  float spatial_scale;
  long count;
};

__global__ __launch_bounds__(256) void roi_pool_kernel(const RoiArgs a) {
  for (long i = blockIdx.x * 256L + threadIdx.x; i < a.count; i += gridDim.x * 256L) {
    const int pw = static_cast<int>(i % a.pooled_w);
    const int ph = static_cast<int>((i / a.pooled_w) % a.pooled_h);
    const int c = static_cast<int>((i / a.pooled_w / a.pooled_h) % a.channels);
    const int n = static_cast<int>(i / a.pooled_w / a.pooled_h / a.channels);
    const float* roi = a.rois + 5 * n;
    const int batch = static_cast<int>(roi[0]);
    if (batch < 0 || batch >= a.num) {
      if (a.bad_flag) *a.bad_flag = 1;
      a.top[i] = 0.f;
      continue;
    }
    const int roi_start_w = static_cast<int>(round(static_cast<double>(roi[1] * a.spatial_scale)));
    const int roi_start_h = static_cast<int>(round(static_cast<double>(roi[2] * a.spatial_scale)));
    const int roi_end_w = static_cast<int>(round(static_cast<double>(roi[3] * a.spatial_scale)));
    const int roi_end_h = static_cast<int>(round(static_cast<double>(roi[4] * a.spatial_scale)));
    const int roi_height = max(roi_end_h - roi_start_h + 1, 1);
    const int roi_width = max(roi_end_w - roi_start_w + 1, 1);
    const float bin_size_h = static_cast<float>(roi_height) / static_cast<float>(a.pooled_h);
    const float bin_size_w = static_cast<float>(roi_width) / static_cast<float>(a.pooled_w);
    int hstart = static_cast<int>(floorf(static_cast<float>(ph) * bin_size_h));
    int wstart = static_cast<int>(floorf(static_cast<float>(pw) * bin_size_w));
    int hend = static_cast<int>(ceilf(static_cast<float>(ph + 1) * bin_size_h));
    int wend = static_cast<int>(ceilf(static_cast<float>(pw + 1) * bin_size_w));
    hstart = min(max(hstart + roi_start_h, 0), a.height);
    hend = min(max(hend + roi_start_h, 0), a.height);
    wstart = min(max(wstart + roi_start_w, 0), a.width);
    wend = min(max(wend + roi_start_w, 0), a.width);
    const bool is_empty = (hend <= hstart) || (wend <= wstart);
    const float* plane = a.bottom + (static_cast<long>(batch) * a.channels + c) * a.height * a.width;
    float v = is_empty ? 0.f : -FLT_MAX;
    for (int h = hstart; h < hend; ++h)
      for (int w = wstart; w < wend; ++w) v = fmaxf(v, plane[h * a.width + w]);
    a.top[i] = v;
  }
}

__global__ __launch_bounds__(256) void psroi_pool_kernel(const RoiArgs a) {
  for (long i = blockIdx.x * 256L + threadIdx.x; i < a.count; i += gridDim.x * 256L) {
    const int pw = static_cast<int>(i % a.pooled_w);
    const int ph = static_cast<int>((i / a.pooled_w) % a.pooled_h);
    const int c = static_cast<int>((i / a.pooled_w / a.pooled_h) % a.output_dim);
    const int n = static_cast<int>(i / a.pooled_w / a.pooled_h / a.output_dim);
    const float* roi = a.rois + 5 * n;
    const int batch = static_cast<int>(roi[0]);
    if (batch < 0 || batch >= a.num) {
      if (a.bad_flag) *a.bad_flag = 1;
      a.top[i] = 0.f;
      continue;
    }
    // corners are rounded before scaling; the products are formed in double and
    // narrowed, as round() returns double in the reference's expression
    const float roi_start_w =
        static_cast<float>(round(static_cast<double>(roi[1])) * a.spatial_scale);
    const float roi_start_h =
        static_cast<float>(round(static_cast<double>(roi[2])) * a.spatial_scale);
    const float roi_end_w =
        static_cast<float>(round(static_cast<double>(roi[3] + 1)) * a.spatial_scale);
    const float roi_end_h =
        static_cast<float>(round(static_cast<double>(roi[4] + 1)) * a.spatial_scale);
    const float roi_height = fmaxf(roi_end_h - roi_start_h, 0.1f);
    const float roi_width = fmaxf(roi_end_w - roi_start_w, 0.1f);
    const float bin_size_h = roi_height / static_cast<float>(a.pooled_h);
    const float bin_size_w = roi_width / static_cast<float>(a.pooled_w);
    int hstart = static_cast<int>(floorf(static_cast<float>(ph) * bin_size_h + roi_start_h));
    int wstart = static_cast<int>(floorf(static_cast<float>(pw) * bin_size_w + roi_start_w));
    int hend = static_cast<int>(ceilf(static_cast<float>(ph + 1) * bin_size_h + roi_start_h));
    int wend = static_cast<int>(ceilf(static_cast<float>(pw + 1) * bin_size_w + roi_start_w));
    hstart = min(max(hstart, 0), a.height);
    hend = min(max(hend, 0), a.height);
    wstart = min(max(wstart, 0), a.width);
    wend = min(max(wend, 0), a.width);
    const bool is_empty = (hend <= hstart) || (wend <= wstart);
    const int fm_c = (c * a.group_size + ph) * a.group_size + pw;
    const float* fm = a.bottom + (static_cast<long>(batch) * a.channels + fm_c) * a.height * a.width;
    float out_sum = 0.f;
    for (int h = hstart; h < hend; ++h)
      for (int w = wstart; w < wend; ++w) out_sum += fm[h * a.width + w];
    const int bin_area = (hend - hstart) * (wend - wstart);
    a.top[i] = is_empty ? 0.f : out_sum / static_cast<float>(bin_area);
  }
}

}  // namespace
}  // namespace mchip

using namespace mchip;

extern "C" {

int mcROIPooling(const float* bottom, int num, int channels, int height, int width,
                 const float* rois, int num_rois, int pooled_h, int pooled_w, float spatial_scale,
                 float* top, int* bad_roi_flag, void* stream) {
  MC_REQUIRE(num_rois >= 0, "mcROIPooling: negative roi count");
  MC_REQUIRE(pooled_h > 0, "pooled_h must be > 0");
  MC_REQUIRE(pooled_w > 0, "pooled_w must be > 0");
  MC_REQUIRE(num > 0 && channels > 0 && height > 0 && width > 0, "mcROIPooling: bad extents");
  if (num_rois == 0) return 0;
  MC_REQUIRE(bottom && rois && top, "mcROIPooling: null argument");
  RoiArgs a = {bottom, rois, top, bad_roi_flag, num, channels, height, width, pooled_h, pooled_w,
               0, 0, spatial_scale, (long)num_rois * channels * pooled_h * pooled_w};
  roi_pool_kernel<<<ew_blocks(a.count, 256), 256, 0, static_cast<hipStream_t>(stream)>>>(a);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcPSROIPooling(const float* bottom, int num, int output_dim, int group_size, int height,
                   int width, const float* rois, int num_rois, float spatial_scale, float* top,
                   int* bad_roi_flag, void* stream) {
  MC_REQUIRE(num_rois >= 0, "mcPSROIPooling: negative roi count");
  MC_REQUIRE(output_dim > 0, "output_dim must be > 0");
  MC_REQUIRE(group_size > 0, "group_size must be > 0");
  MC_REQUIRE(num > 0 && height > 0 && width > 0, "mcPSROIPooling: bad extents");
  if (num_rois == 0) return 0;
  MC_REQUIRE(bottom && rois && top, "mcPSROIPooling: null argument");
  RoiArgs a = {bottom, rois, top, bad_roi_flag, num, output_dim * group_size * group_size, height,
               width, group_size, group_size, group_size, output_dim, spatial_scale,
               (long)num_rois * output_dim * group_size * group_size};
  psroi_pool_kernel<<<ew_blocks(a.count, 256), 256, 0, static_cast<hipStream_t>(stream)>>>(a);
  MC_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
