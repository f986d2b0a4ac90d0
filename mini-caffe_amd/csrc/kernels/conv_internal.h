// Internal interface between the contraction plan (conv_igemm.hip), the direct
// depthwise kernel (conv_depthwise.hip) and the Winograd path (conv_winograd.hip).
#ifndef MCHIP_CONV_INTERNAL_H_
#define MCHIP_CONV_INTERNAL_H_

#include <hip/hip_runtime.h>

#include "mchip/kernels.h"

namespace mchip {

struct DepthwiseArgs {
  const float* x;        // [num, C, H, W]
  const float* w;        // [C * mult, 1, kh, kw] exactly as the layer stores it
  float* y;              // [num, C * mult, Ho, Wo]
  const float* scale;    // per output channel or null
  const float* shift;    // per output channel or null
  const float* residual; // like y or null
  int num, C, mult, H, W, Ho, Wo;
  int kh, kw, sh, sw, ph, pw, dh, dw;
  int act;
  float slope;
};

// y[n][c*mult+j][ho][wo] = act((sum over taps w * x) * scale + shift + residual).
int depthwise_forward(const DepthwiseArgs& a, hipStream_t stream);

// 3x3 stride-1 convolution as F(2x2, 3x3) Winograd: input transform, sixteen
// grouped 1x1 contractions on the implicit-GEMM kernel, output transform with
// the layer's epilogue.  winograd_create returns null for any other geometry.
struct WinogradState;
WinogradState* winograd_create(const mcConvGeom& geom, int Ho, int Wo);
void winograd_destroy(WinogradState* w);
int winograd_set_weights(WinogradState* w, const float* weights, hipStream_t stream);
bool winograd_fits(const WinogradState* w, int num);  // intermediates addressable
bool winograd_pays(const WinogradState* w, int num);  // the automatic choice
double winograd_issued_flops(const WinogradState* w, int num);  // of the sixteen products
int winograd_set_run_bytes(long bytes);  // budget for V + M of one run of images
// top_second / c_first as in mcConvForwardTwoTops (null / ignored for one top)
int winograd_forward(WinogradState* w, int num, const float* bottom, float* top,
                     const mcEpilogue* ep, void* stream, float* top_second, int c_first);

}  // namespace mchip

#endif  // MCHIP_CONV_INTERNAL_H_
