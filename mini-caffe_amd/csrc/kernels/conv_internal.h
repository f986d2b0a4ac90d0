// Internal interface between the contraction plan (conv_igemm.hip) and the
// direct depthwise kernel (conv_depthwise.hip).
#ifndef MCHIP_CONV_INTERNAL_H_
#define MCHIP_CONV_INTERNAL_H_

#include <hip/hip_runtime.h>

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

}  // namespace mchip

#endif  // MCHIP_CONV_INTERNAL_H_
