// 3x3 stride-1 convolution through the Winograd minimal-filtering identity
// F(2x2, 3x3): a 2x2 block of outputs of one channel pair needs 16 products
// instead of 36,
//
//     Y = A^T [ (G g G^T) .* (B^T d B) ] A,
//
// d the 4x4 input patch under the block, g the 3x3 filter.  Summed over the
// input channels the element-wise products are sixteen independent matrix
// products  M_f[Cout][T] = U_f[Cout][Cin] * V_f[Cin][T]  (f = position in the
// 4x4 transform, T = 2x2 output blocks of the whole batch), which is exactly a
// 1x1 convolution with sixteen groups: it runs on the implicit-GEMM kernel of
// conv_igemm.hip through the plan interface.  Three launches per layer:
//
//   winograd_input_kernel    bottom [N, C, H, W]        -> V [16, C, Tpad]
//   igemm (pointwise, g=16)  V, U                       -> M [16, Cout, Tpad]
//   winograd_output_kernel   M (+ scale/shift/residual) -> top [N, Cout, Ho, Wo]
//
// V and M are four times the size of bottom and top, so the detour pays where
// the contraction dominates the traffic: many channels on both sides.  Replaces
// the same reference code as the direct path (conv_layer.cu:7-22 with
// base_conv_layer.cpp:254-278); sums are associated differently from a direct
// convolution (transformed operands, K order over input channels only), within
// the usual fp32 rounding of either.
#include "conv_internal.h"
#include "mc_common.h"
#include "mchip/kernels.h"

#include <algorithm>

namespace mchip {

namespace {

// Channels a thread of a transform kernel walks with one decomposition of its
// block index: four where the launch still has a few workgroups per CU, fewer on
// small maps (7x7 maps of 64 images are 1024 blocks: four workgroups per channel
// group), so that the launch keeps enough loads in flight.
inline int channels_per_thread(long tblocks, int channels, int least) {
  for (int cpt = 4; cpt > least; cpt /= 2)
    if (tblocks * ((channels + cpt - 1) / cpt) >= 8L * kNumCu) return cpt;
  return least;
}

__device__ __forceinline__ float act_value(float v, int act, float slope) {
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

// U[f][co][ci] = (G g G^T)[f / 4][f % 4], G = [1 0 0; 1/2 1/2 1/2; 1/2 -1/2 1/2; 0 0 1].
// One thread per filter.
__global__ __launch_bounds__(256) void winograd_filter_kernel(const float* __restrict__ w,
                                                              float* __restrict__ u, long filters) {
  const long i = blockIdx.x * 256L + threadIdx.x;
  if (i >= filters) return;
  float g[3][3];
#pragma unroll
  for (int r = 0; r < 3; ++r)
#pragma unroll
    for (int c = 0; c < 3; ++c) g[r][c] = w[i * 9 + r * 3 + c];
  float t[4][3];
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    t[0][c] = g[0][c];
    t[1][c] = 0.5f * (g[0][c] + g[1][c] + g[2][c]);
    t[2][c] = 0.5f * (g[0][c] - g[1][c] + g[2][c]);
    t[3][c] = g[2][c];
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    u[(r * 4 + 0) * filters + i] = t[r][0];
    u[(r * 4 + 1) * filters + i] = 0.5f * (t[r][0] + t[r][1] + t[r][2]);
    u[(r * 4 + 2) * filters + i] = 0.5f * (t[r][0] - t[r][1] + t[r][2]);
    u[(r * 4 + 3) * filters + i] = t[r][2];
  }
}

struct WinogradShape {
  int C, H, W, Cout, Ho, Wo, pad_h, pad_w;
  int Th, Tw;       // 2x2 output blocks per image, down and across
  int T, Tpad;      // blocks of the batch; columns of V and M
};

// V[f][c][t] = (B^T d B)[f / 4][f % 4], B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1];
// d = the 4x4 patch of channel c whose corner is output block t's corner minus
// the padding (zeros outside the map).  Lanes run along t, so the sixteen stores
// of a channel are contiguous rows; a thread walks kChannelsPerThread channels
// with one decomposition of t.
template <int CPT>
__global__ __launch_bounds__(256) void winograd_input_kernel(const float* __restrict__ x,
                                                             float* __restrict__ v,
                                                             const WinogradShape s) {
  constexpr int kChannelsPerThread = CPT;
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= s.Tpad) return;
  const int c0 = blockIdx.y * kChannelsPerThread;
  const long fstride = (long)s.C * s.Tpad;
  if (t >= s.T) {
    for (int c = c0; c < min(c0 + kChannelsPerThread, s.C); ++c)
#pragma unroll
      for (int f = 0; f < 16; ++f) v[f * fstride + (long)c * s.Tpad + t] = 0.f;
    return;
  }
  const int per_image = s.Th * s.Tw;
  const int n = t / per_image;
  const int rem = t - n * per_image;
  const int ty = rem / s.Tw;
  const int tx = rem - ty * s.Tw;
  const int h0 = 2 * ty - s.pad_h, w0 = 2 * tx - s.pad_w;
  bool row_ok[4], col_ok[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    row_ok[i] = static_cast<unsigned>(h0 + i) < static_cast<unsigned>(s.H);
    col_ok[i] = static_cast<unsigned>(w0 + i) < static_cast<unsigned>(s.W);
  }
  for (int c = c0; c < min(c0 + kChannelsPerThread, s.C); ++c) {
    const float* plane = x + ((long)n * s.C + c) * s.H * s.W;
    float d[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        d[i][j] = (row_ok[i] && col_ok[j]) ? plane[(h0 + i) * s.W + w0 + j] : 0.f;
    float r[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      r[0][j] = d[0][j] - d[2][j];
      r[1][j] = d[1][j] + d[2][j];
      r[2][j] = d[2][j] - d[1][j];
      r[3][j] = d[1][j] - d[3][j];
    }
    float* out = v + (long)c * s.Tpad + t;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[(i * 4 + 0) * fstride] = r[i][0] - r[i][2];
      out[(i * 4 + 1) * fstride] = r[i][1] + r[i][2];
      out[(i * 4 + 2) * fstride] = r[i][2] - r[i][1];
      out[(i * 4 + 3) * fstride] = r[i][1] - r[i][3];
    }
  }
}

struct WinogradEpilogue {
  const float* scale;
  const float* shift;
  const float* residual;
  int act;
  float slope;
  // two sibling layers computed together: channels [0, c_first) of every image go
  // to the first top [N, c_first, Ho, Wo], the others to y_second; one top: c_first = Cout
  float* y_second;
  int c_first;
};

// Y = A^T m A, A^T = [1 1 1 0; 0 1 -1 -1], m[f] = M[f][co][t]; then the layer's
// epilogue  act(Y * scale[co] + shift[co] + residual)  on the up to four outputs
// of block t that lie inside the map.
template <bool PAIRS, int CPT>
__global__ __launch_bounds__(256) void winograd_output_kernel(const float* __restrict__ m,
                                                              float* __restrict__ y,
                                                              const WinogradShape s,
                                                              const WinogradEpilogue e) {
  constexpr int kChannelsPerThread = CPT;
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= s.T) return;
  const int c0 = blockIdx.y * kChannelsPerThread;
  const long fstride = (long)s.Cout * s.Tpad;
  const int per_image = s.Th * s.Tw;
  const int n = t / per_image;
  const int rem = t - n * per_image;
  const int ty = rem / s.Tw;
  const int tx = rem - ty * s.Tw;
  const int ho = 2 * ty, wo = 2 * tx;
  const bool row1 = ho + 1 < s.Ho, col1 = wo + 1 < s.Wo;
  for (int c = c0; c < min(c0 + kChannelsPerThread, s.Cout); ++c) {
    const float* in = m + (long)c * s.Tpad + t;
    float q[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) q[i][j] = in[(i * 4 + j) * fstride];
    float a[2][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      a[0][j] = q[0][j] + q[1][j] + q[2][j];
      a[1][j] = q[1][j] - q[2][j] - q[3][j];
    }
    float out[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      out[i][0] = a[i][0] + a[i][1] + a[i][2];
      out[i][1] = a[i][1] - a[i][2] - a[i][3];
    }
    const float sc = e.scale ? e.scale[c] : 1.f;
    const float sh = e.shift ? e.shift[c] : 0.f;
    const bool first = c < e.c_first;
    float* __restrict__ yc = first ? y : e.y_second;
    const long base = first ? (((long)n * e.c_first + c) * s.Ho + ho) * s.Wo + wo
                            : (((long)n * (s.Cout - e.c_first) + (c - e.c_first)) * s.Ho + ho) * s.Wo + wo;
    if (e.scale) {
#pragma unroll
      for (int i = 0; i < 2; ++i) out[i][0] *= sc, out[i][1] *= sc;
    }
    if (e.shift) {
#pragma unroll
      for (int i = 0; i < 2; ++i) out[i][0] += sh, out[i][1] += sh;
    }
    if (PAIRS) {
      // even width: a block's two outputs of a row are one aligned 8-byte access
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (i == 1 && !row1) break;
        const long o = base + i * s.Wo;
        float2 val = make_float2(out[i][0], out[i][1]);
        if (e.residual) {
          const float2 r = *reinterpret_cast<const float2*>(e.residual + o);
          val.x += r.x;
          val.y += r.y;
        }
        val.x = act_value(val.x, e.act, e.slope);
        val.y = act_value(val.y, e.act, e.slope);
        *reinterpret_cast<float2*>(yc + o) = val;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (i == 1 && !row1) break;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (j == 1 && !col1) break;
          const long o = base + i * s.Wo + j;
          float val = out[i][j];
          if (e.residual) val += e.residual[o];
          yc[o] = act_value(val, e.act, e.slope);
        }
      }
    }
  }
}

}  // namespace

struct WinogradState {
  mcConvGeom geom;
  int Ho = 0, Wo = 0;
  float* u = nullptr;          // transformed filters [16 * Cout, Cin]
  bool have_weights = false;
  // 1x1 plans with sixteen groups on a one-image blob of Tpad pixels, by Tpad: a
  // batch runs in at most two different run lengths
  struct Inner {
    int tpad = 0;
    mcConvPlan* plan = nullptr;
  };
  Inner inner[2];
  int next_inner = 0;
};

// Bytes of V and M one run of images may take; a larger batch is cut into equal
// runs of whole images.  It bounds the workspace, nothing else: shorter runs that
// keep V and M in the last-level cache were measured and are slower (every run
// pays the ramp and tail of three launches).
long g_winograd_run_bytes = 1L << 30;

bool winograd_eligible(const mcConvGeom& g) {
  return !g.transposed && g.group == 1 && g.kernel_h == 3 && g.kernel_w == 3 && g.stride_h == 1 &&
         g.stride_w == 1 && g.dilation_h == 1 && g.dilation_w == 1 && g.pad_h <= 2 && g.pad_w <= 2;
}

WinogradState* winograd_create(const mcConvGeom& g, int Ho, int Wo) {
  if (!winograd_eligible(g)) return nullptr;
  WinogradState* w = new WinogradState();
  w->geom = g;
  w->Ho = Ho;
  w->Wo = Wo;
  return w;
}

void winograd_destroy(WinogradState* w) {
  if (!w) return;
  for (auto& in : w->inner)
    if (in.plan) (void)mcConvPlanDestroy(in.plan);
  if (w->u) (void)hipFree(w->u);
  delete w;
}

namespace {
// The contraction sees V as a one-image blob of `rows` x (Tpad / rows) pixels; both
// extents stay below its limit of 16384, and a row is a multiple of four pixels
// (16-byte gathers).
inline long plane_rows(long T) { return (T + 8191) / 8192; }
inline long padded_blocks(long T) {
  const long unit = 4 * plane_rows(T);
  return (T + unit - 1) / unit * unit;
}

WinogradShape shape_of(const WinogradState* w, int num) {
  WinogradShape s;
  s.C = w->geom.channels_in;
  s.H = w->geom.height_in;
  s.W = w->geom.width_in;
  s.Cout = w->geom.channels_out;
  s.Ho = w->Ho;
  s.Wo = w->Wo;
  s.pad_h = w->geom.pad_h;
  s.pad_w = w->geom.pad_w;
  s.Th = (w->Ho + 1) / 2;
  s.Tw = (w->Wo + 1) / 2;
  const long T = (long)num * s.Th * s.Tw;
  s.T = static_cast<int>(T);
  s.Tpad = static_cast<int>(padded_blocks(T));
  return s;
}
}  // namespace

// Whether a batch of `num` images can take this path at all: V and M must stay
// below the 2^29 elements one contraction launch addresses.
bool winograd_fits(const WinogradState* w, int num) {
  const long blocks = (long)num * ((w->Ho + 1) / 2) * ((w->Wo + 1) / 2);
  const long T = padded_blocks(blocks);
  const long most = 16L * std::max(w->geom.channels_in, w->geom.channels_out) * T;
  // (the transform kernels put channels on the grid's y axis)
  return plane_rows(blocks) < 16384 && most < (1L << 29) &&
         std::max(w->geom.channels_in, w->geom.channels_out) <= 65535;
}

// The automatic choice.  Per output block the direct path multiplies 36 Cin Cout
// times and moves 4 (Cin + Cout) floats; this path multiplies 16 Cin Cout times
// and moves 16 (Cin + Cout) floats twice (V and M, written and read) besides.
// Measured on the 3x3 layers of ResNet-50 (batch 64), VGG-16 / SSD300 (batch 8)
// and an RPN head, direct against this path: 64 channels lose everywhere (151 us
// against 209 on 56x56 maps); 128 -> 128 gains while V and M fit the 256 MB
// last-level cache (152 -> 108 us on 28x28 maps) and loses beyond it (428 -> 478
// on 150x150); 128 -> 256 gains 1.17x; 256 and 512 channels gain 1.4x to 1.8x on
// every map.  One narrow side is fine when the other is wide (SSD's merged heads,
// 512 -> 100 on 38x38 b8: 147 -> 92 us; 1024 -> 150 on 19x19: 113 -> 81; 96 -> 512:
// 91 -> 76) down to about 96 channels (256 -> 64 and 64 -> 512 break even, 1024 ->
// 64 loses); 200 blocks still gain or break even (512 -> 150 on 10x10 b8: 42 -> 30 us).
bool winograd_pays(const WinogradState* w, int num) {
  const mcConvGeom& g = w->geom;
  const long blocks = (long)num * ((w->Ho + 1) / 2) * ((w->Wo + 1) / 2);
  const int least = std::min(g.channels_in, g.channels_out);
  const int most = std::max(g.channels_in, g.channels_out);
  if (blocks < 192 || least < 96) return false;
  // odd and tiny maps compute blocks that hang over the edge: a 3x3 map is four
  // blocks for nine outputs (16 x 4 products against 36 x 9 / 4 useful ones)
  if (10L * w->Ho * w->Wo < 26L * ((w->Ho + 1) / 2) * ((w->Wo + 1) / 2)) return false;
  if (most >= 256) return true;
  return least >= 128 && 64L * (g.channels_in + g.channels_out) * blocks <= (256L << 20);
}

int winograd_set_weights(WinogradState* w, const float* weights, hipStream_t st) {
  const long filters = (long)w->geom.channels_out * w->geom.channels_in;
  if (!w->u) MC_HIP(hipMalloc(&w->u, sizeof(float) * 16 * filters));
  winograd_filter_kernel<<<ew_blocks(filters, 256), 256, 0, st>>>(weights, w->u, filters);
  MC_LAUNCH_CHECK();
  w->have_weights = true;
  for (auto& in : w->inner)
    if (in.plan && mcConvPlanSetWeights(in.plan, w->u, st)) return -1;
  return 0;
}

namespace {
int inner_plan(WinogradState* w, const WinogradShape& s, hipStream_t st, mcConvPlan** out) {
  for (auto& in : w->inner)
    if (in.plan && in.tpad == s.Tpad) {
      *out = in.plan;
      return 0;
    }
  WinogradState::Inner& slot = w->inner[w->next_inner];
  w->next_inner ^= 1;
  if (slot.plan) {
    // kernels of an earlier call may still read the old plan's filter copy
    MC_HIP(hipStreamSynchronize(st));
    (void)mcConvPlanDestroy(slot.plan);
    slot.plan = nullptr;
  }
  mcConvGeom g;
  g.channels_in = 16 * s.C;
  g.height_in = static_cast<int>(plane_rows(s.T));
  g.width_in = s.Tpad / g.height_in;
  g.channels_out = 16 * s.Cout;
  g.kernel_h = g.kernel_w = 1;
  g.stride_h = g.stride_w = 1;
  g.pad_h = g.pad_w = 0;
  g.dilation_h = g.dilation_w = 1;
  g.group = 16;
  g.transposed = 0;
  if (mcConvPlanCreate(&g, &slot.plan)) return -1;
  slot.tpad = s.Tpad;
  if (mcConvPlanSetWeights(slot.plan, w->u, st)) return -1;
  *out = slot.plan;
  return 0;
}
}  // namespace

double winograd_issued_flops(const WinogradState* w, int num) {
  const double blocks = (double)num * ((w->Ho + 1) / 2) * ((w->Wo + 1) / 2);
  return 2. * 16. * w->geom.channels_in * w->geom.channels_out * blocks;
}

int winograd_set_run_bytes(long bytes) {
  g_winograd_run_bytes = std::max(bytes, 1L << 20);
  return 0;
}

int winograd_forward(WinogradState* w, int num, const float* bottom, float* top,
                     const mcEpilogue* ep, void* stream, float* top_second, int c_first) {
  MC_REQUIRE(w->have_weights, "mcConvForward: the plan has no weights yet");
  MC_REQUIRE(!top_second || (c_first > 0 && c_first < w->geom.channels_out && !(ep && ep->residual)),
             "mcConvForwardTwoTops: needs group 1, a split inside the output channels and no "
             "residual");
  if (!top_second) c_first = w->geom.channels_out;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const mcConvGeom& g = w->geom;
  // equal runs of whole images whose V and M fit the budget
  const long per_image =
      64L * (g.channels_in + g.channels_out) * ((w->Ho + 1) / 2) * ((w->Wo + 1) / 2);
  const long fit = std::max(1L, g_winograd_run_bytes / per_image);
  const int runs = ceil_div(num, fit);
  const int run_len = ceil_div(num, runs);
  const long in_img = (long)g.channels_in * g.height_in * g.width_in;
  const long hw_out = (long)w->Ho * w->Wo;
  const long out_img = c_first * hw_out, second_img = (g.channels_out - c_first) * hw_out;
  WinogradEpilogue e;
  e.c_first = c_first;
  e.scale = ep ? ep->scale : nullptr;
  e.shift = ep ? ep->shift : nullptr;
  e.act = ep ? ep->activation : MC_ACT_NONE;
  e.slope = ep ? ep->negative_slope : 0.f;
  for (int n0 = 0; n0 < num; n0 += run_len) {
    const int n = std::min(run_len, num - n0);
    const WinogradShape s = shape_of(w, n);
    mcConvPlan* inner = nullptr;
    if (inner_plan(w, s, st, &inner)) return -1;
    float* ws = nullptr;
    const size_t v_floats = 16ul * s.C * s.Tpad, m_floats = 16ul * s.Cout * s.Tpad;
    if (stream_workspace(st, sizeof(float) * (v_floats + m_floats), &ws, 1)) return -1;
    float* v = ws;
    float* m = ws + v_floats;
    const unsigned tblocks = static_cast<unsigned>(ceil_div(s.Tpad, 256));
    const float* run_bottom = bottom + n0 * in_img;
    float* run_top = top + n0 * out_img;
    switch (channels_per_thread(tblocks, s.C, 1)) {
      case 4:
        winograd_input_kernel<4><<<dim3(tblocks, ceil_div(s.C, 4)), 256, 0, st>>>(run_bottom, v, s);
        break;
      case 2:
        winograd_input_kernel<2><<<dim3(tblocks, ceil_div(s.C, 2)), 256, 0, st>>>(run_bottom, v, s);
        break;
      default:
        winograd_input_kernel<1><<<dim3(tblocks, s.C), 256, 0, st>>>(run_bottom, v, s);
    }
    MC_LAUNCH_CHECK();
    if (mcConvForward(inner, 1, v, m, nullptr, stream)) return -1;
    e.residual = (ep && ep->residual) ? ep->residual + n0 * out_img : nullptr;
    const unsigned oblocks = static_cast<unsigned>(ceil_div(s.T, 256));
    // (top and residual rows are 8-byte aligned when the width is even and the blob is)
    e.y_second = top_second ? top_second + n0 * second_img : nullptr;
    const bool pairs = s.Wo % 2 == 0 && reinterpret_cast<uintptr_t>(top) % 8 == 0 &&
                       reinterpret_cast<uintptr_t>(top_second) % 8 == 0 &&
                       (!ep || !ep->residual || reinterpret_cast<uintptr_t>(ep->residual) % 8 == 0);
    const int cpt = channels_per_thread(oblocks, s.Cout, 2);  // (one channel per thread measured slower here)
    const dim3 ogrid(oblocks, ceil_div(s.Cout, cpt));
#define MC_WINOGRAD_OUT(P, C) winograd_output_kernel<P, C><<<ogrid, 256, 0, st>>>(m, run_top, s, e)
    if (pairs) {
      if (cpt == 4) MC_WINOGRAD_OUT(true, 4);
      else MC_WINOGRAD_OUT(true, 2);
    } else {
      if (cpt == 4) MC_WINOGRAD_OUT(false, 4);
      else MC_WINOGRAD_OUT(false, 2);
    }
#undef MC_WINOGRAD_OUT
    MC_LAUNCH_CHECK();
  }
  return 0;
}

}  // namespace mchip
