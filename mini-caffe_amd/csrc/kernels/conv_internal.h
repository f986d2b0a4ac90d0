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

// Multiplier and shift with  n / d == mulhi(n, mul) >> shift  for 0 <= n < n_max.
// shift 32 stands for d == 1 (no 32-bit multiplier exists for it).
inline void make_fast_div(unsigned d, unsigned long long n_max, unsigned* mul, unsigned* shift) {
  *mul = 0;
  *shift = 32;
  if (d <= 1) return;
  for (int s = 31; s >= 0; --s) {
    const unsigned __int128 pow = (unsigned __int128)1 << (32 + s);
    const unsigned __int128 m = (pow + d - 1) / d;
    if (m >> 32) continue;
    const unsigned __int128 err = m * d - pow;  // 0 <= err < d
    if (err * n_max < pow) {
      *mul = static_cast<unsigned>(m);
      *shift = static_cast<unsigned>(s);
      return;
    }
  }
  // unreachable for n_max < 2^32: s = 0 gives err * n_max < d * 2^32 / d
}

// n / d for the d the host prepared (mul, shift) for; shift == 32 means d == 1.
__device__ __forceinline__ int fast_div(int n, unsigned mul, unsigned shift) {
  // both sides computed and picked by a mask: as a conditional expression on the uniform
  // `shift` this becomes a branch, which splits a kernel's prologue into blocks and
  // leaves its argument loads waiting one after the other
  const unsigned q = __umulhi(static_cast<unsigned>(n), mul) >> (shift & 31);
  const unsigned keep = shift == 32 ? 0xFFFFFFFFu : 0u;
  return static_cast<int>((static_cast<unsigned>(n) & keep) | (q & ~keep));
}

// 3x3 stride-1 convolution as F(2x2, 3x3) Winograd in one launch: the input
// transform in the loader, the sixteen products on the matrix cores, the output
// transform and the layer's epilogue before the store.  winograd_create returns
// null for any other geometry.
struct WinogradState;
WinogradState* winograd_create(const mcConvGeom& geom, int Ho, int Wo);
void winograd_destroy(WinogradState* w);
int winograd_set_weights(WinogradState* w, const float* weights, hipStream_t stream);
bool winograd_fits(const WinogradState* w, int num);  // one image addressable by the kernel
bool winograd_pays(const WinogradState* w, int num);  // the automatic choice
double winograd_issued_flops(const WinogradState* w, int num);  // of the sixteen products
// top_second / c_first as in mcConvForwardTwoTops (null / ignored for one top);
// images_per_run > 0 caps the images one launch takes, forced_slices > 0 fixes the
// number of slices the input channels are cut into
int winograd_forward(WinogradState* w, int num, const float* bottom, float* top,
                     const mcEpilogue* ep, void* stream, float* top_second, int c_first,
                     int images_per_run, int forced_slices);

}  // namespace mchip

#endif  // MCHIP_CONV_INTERNAL_H_
