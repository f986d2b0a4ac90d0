// HBM-bound per-channel and elementwise kernels: the fused BatchNorm / Scale /
// Bias / activation pass, BatchNorm statistics, Eltwise, fill and strided copy.
//
// All of them move each element once: one global read per input and one global
// write per output, 16-byte vector accesses whenever the shape allows it, and a
// grid of a few waves per CU walking the blob with a grid stride.
#include <algorithm>

#include "mc_common.h"
#include "mchip/kernels.h"

#include <cfloat>

namespace mchip {
namespace {

__device__ __forceinline__ float act_apply(float v, int act, float slope) {
  switch (act) {
    case MC_ACT_RELU:
      // slope == 0 gives max(x,0); otherwise max(x,0) + slope*min(x,0)
      // (reference relu_layer.cpp:18-28).
      return v > 0.f ? v : v * slope;
    case MC_ACT_TANH:
      return static_cast<float>(tanh(static_cast<double>(v)));
    case MC_ACT_SIGMOID:
      return static_cast<float>(1. / (1. + exp(-static_cast<double>(v))));
    default:
      return v;
  }
}

struct ChanArgs {
  const float* __restrict__ x;
  float* __restrict__ y;
  const float* __restrict__ sub;
  const float* __restrict__ div;
  const float* __restrict__ mul;
  const float* __restrict__ add;
  long count;     // outer*channels*inner
  int channels;
  int inner;
  int act;
  float slope;
};

// The channel's four operands, fetched once per vector (absent ones are the
// neutral element), then  ((v - sub) / div) * mul + add  and the activation.
// TRANS = false compiles only "none" and ReLU: the double-precision tanh / exp
// of the other two activations would otherwise sit in the loop of every launch.
template <bool TRANS>
__device__ __forceinline__ float chan_one(float v, float sub, float div, float mul, float add,
                                          bool has_div, const ChanArgs& a) {
  v -= sub;
  if (has_div) v /= div;
  v = v * mul + add;
  if (TRANS) return act_apply(v, a.act, a.slope);
  return (a.act == MC_ACT_RELU && !(v > 0.f)) ? v * a.slope : v;
}

// VEC = 4 requires inner % 4 == 0, so the four lanes of a float4 share a channel.
template <int VEC, bool TRANS>
__global__ __launch_bounds__(256) void channel_transform_kernel(const ChanArgs a) {
  const long n = a.count / VEC;
  const bool has_div = a.div != nullptr;
  for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += gridDim.x * 256L) {
    const long e = i * VEC;
    const int c = static_cast<int>((e / a.inner) % a.channels);
    const float sub = a.sub ? a.sub[c] : 0.f, div = has_div ? a.div[c] : 1.f;
    const float mul = a.mul ? a.mul[c] : 1.f, add = a.add ? a.add[c] : 0.f;
    if (VEC == 4) {
      float4 v = reinterpret_cast<const float4*>(a.x)[i];
      v.x = chan_one<TRANS>(v.x, sub, div, mul, add, has_div, a);
      v.y = chan_one<TRANS>(v.y, sub, div, mul, add, has_div, a);
      v.z = chan_one<TRANS>(v.z, sub, div, mul, add, has_div, a);
      v.w = chan_one<TRANS>(v.w, sub, div, mul, add, has_div, a);
      reinterpret_cast<float4*>(a.y)[i] = v;
    } else {
      a.y[i] = chan_one<TRANS>(a.x[i], sub, div, mul, add, has_div, a);
    }
  }
}

__global__ void bn_stored_kernel(const float* __restrict__ b0, const float* __restrict__ b1,
                                 const float* __restrict__ b2, float eps, int C,
                                 float* __restrict__ mean, float* __restrict__ stdev) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const float f = b2[0] == 0.f ? 0.f : 1.f / b2[0];
  mean[c] = f * b0[c];
  stdev[c] = sqrtf(f * b1[c] + eps);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
__device__ __forceinline__ float block_sum(float v, float* lds16) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds16[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.f;
  for (int w = 0; w < static_cast<int>(blockDim.x >> 6); ++w) t += lds16[w];
  return t;
}

// Batch statistics of one channel: mean, then the mean of squared deviations, as
// two passes over the values (the second pass re-reads them from cache).  A
// workgroup (up to 1024 threads) takes the images [blockIdx.y * per, + per) of
// channel blockIdx.x.  With one part per channel it writes mean and deviation
// itself; otherwise it leaves {mean, sum of squared deviations from that mean}
// of its part in `partial`, and bn_batch_combine_kernel merges the parts (the
// parallel form of the two-pass variance: M2 = sum M2_i + sum n_i (m_i - m)^2).
// VEC = 4 walks each image's plane with float4 loads; the (image, position) pair
// of a thread advances by a fixed step, so the loops hold no division.
template <int VEC>
__global__ __launch_bounds__(1024) void bn_batch_stats_kernel(const float* __restrict__ x, int num,
                                                              int C, int spatial, float eps,
                                                              float* __restrict__ mean,
                                                              float* __restrict__ stdev, int per,
                                                              float2* __restrict__ partial) {
  __shared__ float red[16];
  const int c = blockIdx.x;
  const int first = blockIdx.y * per;
  const int last = min(first + per, num);  // images [first, last)
  const int per_row = spatial / VEC;       // vectors per image plane
  const int step_n = blockDim.x / per_row, step_v = blockDim.x % per_row;
  const int n0 = first + threadIdx.x / per_row, v0 = threadIdx.x % per_row;
  const float alpha = static_cast<float>(1. / (static_cast<double>(last - first) * spatial));
  const long plane = spatial, image = (long)C * spatial;
  const float* __restrict__ xc = x + c * plane;
  float s = 0.f;
  for (int n = n0, v = v0; n < last;) {
    const float* p = xc + n * image + v * VEC;
    if (VEC == 4) {
      const float4 t = *reinterpret_cast<const float4*>(p);
      s += (t.x + t.y) + (t.z + t.w);
    } else {
      s += *p;
    }
    n += step_n;
    v += step_v;
    if (v >= per_row) {
      v -= per_row;
      ++n;
    }
  }
  const float m = alpha * block_sum(s, red);
  float q = 0.f;
  for (int n = n0, v = v0; n < last;) {
    const float* p = xc + n * image + v * VEC;
    if (VEC == 4) {
      const float4 t = *reinterpret_cast<const float4*>(p);
      const float d0 = t.x - m, d1 = t.y - m, d2 = t.z - m, d3 = t.w - m;
      q += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
    } else {
      const float d = *p - m;
      q += d * d;
    }
    n += step_n;
    v += step_v;
    if (v >= per_row) {
      v -= per_row;
      ++n;
    }
  }
  const float m2 = block_sum(q, red);
  if (threadIdx.x == 0) {
    if (partial) {
      partial[c * gridDim.y + blockIdx.y] = make_float2(m, m2);
    } else {
      mean[c] = m;
      stdev[c] = sqrtf(alpha * m2 + eps);
    }
  }
}

// One thread per channel merges the parts of bn_batch_stats_kernel, in part order.
__global__ __launch_bounds__(256) void bn_batch_combine_kernel(const float2* __restrict__ partial,
                                                               int parts, int per, int num, int C,
                                                               int spatial, float eps,
                                                               float* __restrict__ mean,
                                                               float* __restrict__ stdev) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const float total = static_cast<float>(num) * spatial;
  float m = 0.f;
  for (int z = 0; z < parts; ++z) {
    const float n_z = static_cast<float>(min(per, num - z * per)) * spatial;
    m += partial[c * parts + z].x * (n_z / total);
  }
  float m2 = 0.f;
  for (int z = 0; z < parts; ++z) {
    const float n_z = static_cast<float>(min(per, num - z * per)) * spatial;
    const float2 t = partial[c * parts + z];
    const float d = t.x - m;
    m2 += t.y + n_z * d * d;
  }
  mean[c] = m;
  stdev[c] = sqrtf(m2 / total + eps);
}

struct FoldArgs {
  const float* bias0;
  mcChannelOp st[4];
  int ns;
  int C;
  float* scale;
  float* shift;
};

__global__ void fold_kernel(const FoldArgs a) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= a.C) return;
  float s = 1.f, t = a.bias0 ? a.bias0[c] : 0.f;
  for (int i = 0; i < a.ns; ++i) {
    const mcChannelOp& o = a.st[i];
    if (o.sub) t -= o.sub[c];
    if (o.div) {
      s /= o.div[c];
      t /= o.div[c];
    }
    if (o.mul) {
      s *= o.mul[c];
      t *= o.mul[c];
    }
    if (o.add) t += o.add[c];
  }
  a.scale[c] = s;
  a.shift[c] = t;
}

struct EltArgs {
  const float* in[8];
  float coeff[8];
  float* out;
  long count;
  int nb;
  int op;
  int act;
  float slope;
};

__device__ __forceinline__ float elt_combine(int op, float acc, float v, float coeff) {
  if (op == MC_ELT_PROD) return acc * v;
  if (op == MC_ELT_SUM) return coeff * v + acc;
  return v > acc ? v : acc;
}

template <int VEC>
__global__ __launch_bounds__(256) void eltwise_kernel(const EltArgs a) {
  const long n = a.count / VEC;
  for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += gridDim.x * 256L) {
    if (VEC == 4) {
      float4 acc;
      if (a.op == MC_ELT_SUM) {
        acc = make_float4(0.f, 0.f, 0.f, 0.f);
      } else {
        acc = reinterpret_cast<const float4*>(a.in[0])[i];
      }
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        if (b >= a.nb) break;
        if (b == 0 && a.op != MC_ELT_SUM) continue;
        const float4 v = reinterpret_cast<const float4*>(a.in[b])[i];
        acc.x = elt_combine(a.op, acc.x, v.x, a.coeff[b]);
        acc.y = elt_combine(a.op, acc.y, v.y, a.coeff[b]);
        acc.z = elt_combine(a.op, acc.z, v.z, a.coeff[b]);
        acc.w = elt_combine(a.op, acc.w, v.w, a.coeff[b]);
      }
      acc.x = act_apply(acc.x, a.act, a.slope);
      acc.y = act_apply(acc.y, a.act, a.slope);
      acc.z = act_apply(acc.z, a.act, a.slope);
      acc.w = act_apply(acc.w, a.act, a.slope);
      reinterpret_cast<float4*>(a.out)[i] = acc;
    } else {
      float acc = a.op == MC_ELT_SUM ? 0.f : a.in[0][i];
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        if (b >= a.nb) break;
        if (b == 0 && a.op != MC_ELT_SUM) continue;
        acc = elt_combine(a.op, acc, a.in[b][i], a.coeff[b]);
      }
      a.out[i] = act_apply(acc, a.act, a.slope);
    }
  }
}

__global__ __launch_bounds__(256) void fill_kernel(float* __restrict__ dst, long count, float v) {
  for (long i = blockIdx.x * 256L + threadIdx.x; i < count; i += gridDim.x * 256L) dst[i] = v;
}

template <int VEC>
__global__ __launch_bounds__(256) void copy2d_kernel(const float* __restrict__ src, long src_pitch,
                                                     float* __restrict__ dst, long dst_pitch,
                                                     long width, long rows) {
  const long wv = width / VEC;
  const long n = wv * rows;
  for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += gridDim.x * 256L) {
    const long r = i / wv, c = (i - r * wv) * VEC;
    if (VEC == 4) {
      *reinterpret_cast<float4*>(dst + r * dst_pitch + c) =
          *reinterpret_cast<const float4*>(src + r * src_pitch + c);
    } else {
      dst[r * dst_pitch + c] = src[r * src_pitch + c];
    }
  }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Up to kConcatSources strided copies into one destination in one launch: blockIdx.y is
// the source, the x extent of the grid covers the largest of them.
constexpr int kConcatSources = 8;
struct ConcatArgs {
  const float* src[kConcatSources];
  long width[kConcatSources];   // floats per row of the source (its pitch as well)
  long offset[kConcatSources];  // where its rows start inside a destination row
  float* dst;
  long dst_pitch, rows;
};
template <int VEC>
__global__ __launch_bounds__(256) void concat_kernel(const ConcatArgs a) {
  const int k = blockIdx.y;
  const float* __restrict__ src = a.src[k];
  float* __restrict__ dst = a.dst + a.offset[k];
  const long wv = a.width[k] / VEC;
  const long n = wv * a.rows;
  for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += gridDim.x * 256L) {
    const long r = i / wv, c = (i - r * wv) * VEC;
    if (VEC == 4) {
      *reinterpret_cast<float4*>(dst + r * a.dst_pitch + c) =
          *reinterpret_cast<const float4*>(src + r * a.width[k] + c);
    } else {
      dst[r * a.dst_pitch + c] = src[r * a.width[k] + c];
    }
  }
}

}  // namespace
}  // namespace mchip

using namespace mchip;

extern "C" {

int mcChannelTransform(const float* x, float* y, int outer, int channels, int inner,
                       const mcChannelOp* op, void* stream) {
  MC_REQUIRE(x && y && op, "mcChannelTransform: null argument");
  MC_REQUIRE(outer >= 0 && channels > 0 && inner > 0, "mcChannelTransform: bad extents");
  ChanArgs a;
  a.x = x;
  a.y = y;
  a.sub = op->sub;
  a.div = op->div;
  a.mul = op->mul;
  a.add = op->add;
  a.count = (long)outer * channels * inner;
  a.channels = channels;
  a.inner = inner;
  a.act = op->activation;
  a.slope = op->negative_slope;
  if (a.count == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool trans = a.act == MC_ACT_TANH || a.act == MC_ACT_SIGMOID;
  if (inner % 4 == 0 && aligned16(x) && aligned16(y)) {
    const int blocks = ew_blocks(a.count / 4, 256);
    if (trans) channel_transform_kernel<4, true><<<blocks, 256, 0, st>>>(a);
    else channel_transform_kernel<4, false><<<blocks, 256, 0, st>>>(a);
  } else {
    const int blocks = ew_blocks(a.count, 256);
    if (trans) channel_transform_kernel<1, true><<<blocks, 256, 0, st>>>(a);
    else channel_transform_kernel<1, false><<<blocks, 256, 0, st>>>(a);
  }
  MC_LAUNCH_CHECK();
  return 0;
}

int mcBatchNormStored(const float* blob0, const float* blob1, const float* blob2, float eps,
                      int channels, float* mean, float* stdev, void* stream) {
  MC_REQUIRE(blob0 && blob1 && blob2 && mean && stdev, "mcBatchNormStored: null argument");
  MC_REQUIRE(channels > 0, "mcBatchNormStored: bad channel count");
  bn_stored_kernel<<<ceil_div(channels, 256), 256, 0, static_cast<hipStream_t>(stream)>>>(
      blob0, blob1, blob2, eps, channels, mean, stdev);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcBatchNormBatchStats(const float* x, int num, int channels, int spatial, float eps,
                          float* mean, float* stdev, void* stream) {
  MC_REQUIRE(x && mean && stdev, "mcBatchNormBatchStats: null argument");
  MC_REQUIRE(num > 0 && channels > 0 && spatial > 0, "mcBatchNormBatchStats: bad extents");
  const bool vec = spatial % 4 == 0 && aligned16(x);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Few channels would leave most of the chip idle: cut each channel's images
  // into parts of at least 4096 values (16384 with float4 loads) until about
  // four workgroups per compute unit exist.
  const long part_min = vec ? 16384 : 4096;
  int parts = 1;
  while (channels * parts < 1024 && parts * 2 <= num && ((long)num / (parts * 2)) * spatial >= part_min) parts *= 2;
  const int per = ceil_div(num, parts);
  parts = ceil_div(num, per);
  float2* partial = nullptr;
  if (parts > 1) {
    float* ws = nullptr;
    if (stream_workspace(st, sizeof(float2) * channels * parts, &ws)) return -1;
    partial = reinterpret_cast<float2*>(ws);
  }
  const long per_part = (long)per * (vec ? spatial / 4 : spatial);
  const int threads = per_part >= 1024 ? 1024 : 256;
  const dim3 grid(channels, parts);
  if (vec)
    bn_batch_stats_kernel<4><<<grid, threads, 0, st>>>(x, num, channels, spatial, eps, mean, stdev, per, partial);
  else
    bn_batch_stats_kernel<1><<<grid, threads, 0, st>>>(x, num, channels, spatial, eps, mean, stdev, per, partial);
  MC_LAUNCH_CHECK();
  if (parts > 1) {
    bn_batch_combine_kernel<<<ceil_div(channels, 256), 256, 0, st>>>(partial, parts, per, num, channels,
                                                                       spatial, eps, mean, stdev);
    MC_LAUNCH_CHECK();
  }
  return 0;
}

int mcFoldChannelOps(const float* bias0, const mcChannelOp* stages, int num_stages, int channels,
                     float* scale, float* shift, void* stream) {
  MC_REQUIRE(scale && shift, "mcFoldChannelOps: null output");
  MC_REQUIRE(num_stages >= 0 && num_stages <= 4, "mcFoldChannelOps: at most 4 stages");
  MC_REQUIRE(num_stages == 0 || stages, "mcFoldChannelOps: null stages");
  FoldArgs a;
  a.bias0 = bias0;
  for (int i = 0; i < num_stages; ++i) a.st[i] = stages[i];
  a.ns = num_stages;
  a.C = channels;
  a.scale = scale;
  a.shift = shift;
  fold_kernel<<<ceil_div(channels, 256), 256, 0, static_cast<hipStream_t>(stream)>>>(a);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcEltwise(int op, int num_bottoms, const float* const* bottoms, const float* coeffs,
              long count, float* top, int activation, float negative_slope, void* stream) {
  MC_REQUIRE(bottoms && top, "mcEltwise: null argument");
  MC_REQUIRE(op >= MC_ELT_PROD && op <= MC_ELT_MAX, "Unknown elementwise operation.");
  MC_REQUIRE(num_bottoms >= 1 && num_bottoms <= 8, "mcEltwise: 1..8 bottoms supported");
  MC_REQUIRE(op == MC_ELT_SUM || num_bottoms >= 2, "mcEltwise: PROD/MAX need two bottoms");
  if (count == 0) return 0;
  EltArgs a;
  bool vec = count % 4 == 0 && aligned16(top);
  for (int i = 0; i < 8; ++i) {
    a.in[i] = i < num_bottoms ? bottoms[i] : nullptr;
    a.coeff[i] = (coeffs && i < num_bottoms) ? coeffs[i] : 1.f;
    if (i < num_bottoms) {
      MC_REQUIRE(bottoms[i], "mcEltwise: null bottom");
      vec = vec && aligned16(bottoms[i]);
    }
  }
  a.out = top;
  a.count = count;
  a.nb = num_bottoms;
  a.op = op;
  a.act = activation;
  a.slope = negative_slope;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (vec) {
    eltwise_kernel<4><<<ew_blocks(count / 4, 256), 256, 0, st>>>(a);
  } else {
    eltwise_kernel<1><<<ew_blocks(count, 256), 256, 0, st>>>(a);
  }
  MC_LAUNCH_CHECK();
  return 0;
}

int mcFill(float* dst, long count, float value, void* stream) {
  MC_REQUIRE(dst || count == 0, "mcFill: null argument");
  if (count <= 0) return 0;
  fill_kernel<<<ew_blocks(count, 256), 256, 0, static_cast<hipStream_t>(stream)>>>(dst, count,
                                                                                    value);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcCopy2D(const float* src, long src_pitch, float* dst, long dst_pitch, long width, long rows,
             void* stream) {
  MC_REQUIRE(src && dst, "mcCopy2D: null argument");
  MC_REQUIRE(width >= 0 && rows >= 0 && src_pitch >= width && dst_pitch >= width,
             "mcCopy2D: bad extents");
  if (width == 0 || rows == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = width % 4 == 0 && src_pitch % 4 == 0 && dst_pitch % 4 == 0 && aligned16(src) &&
                   aligned16(dst);
  if (vec) {
    copy2d_kernel<4><<<ew_blocks(width / 4 * rows, 256), 256, 0, st>>>(src, src_pitch, dst,
                                                                       dst_pitch, width, rows);
  } else {
    copy2d_kernel<1><<<ew_blocks(width * rows, 256), 256, 0, st>>>(src, src_pitch, dst, dst_pitch,
                                                                   width, rows);
  }
  MC_LAUNCH_CHECK();
  return 0;
}

int mcConcat(const float* const* srcs, const long* widths, int count, float* dst, long rows,
             void* stream) {
  MC_REQUIRE(srcs && widths && dst && count > 0 && rows >= 0, "mcConcat: bad argument");
  long pitch = 0;
  for (int i = 0; i < count; ++i) {
    MC_REQUIRE(widths[i] >= 0 && (widths[i] == 0 || srcs[i]), "mcConcat: bad source");
    pitch += widths[i];
  }
  if (rows == 0 || pitch == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  long offset = 0;
  for (int first = 0; first < count; first += kConcatSources) {
    ConcatArgs a;
    a.dst = dst;
    a.dst_pitch = pitch;
    a.rows = rows;
    int n = 0;
    long widest = 0;
    bool vec = pitch % 4 == 0 && aligned16(dst);
    for (int i = first; i < count && i < first + kConcatSources; ++i) {
      if (widths[i] == 0) continue;
      a.src[n] = srcs[i];
      a.width[n] = widths[i];
      a.offset[n] = offset;
      vec = vec && widths[i] % 4 == 0 && offset % 4 == 0 && aligned16(srcs[i]);
      widest = std::max(widest, widths[i]);
      offset += widths[i];
      ++n;
    }
    if (n == 0) continue;
    if (vec)
      concat_kernel<4><<<dim3(ew_blocks(widest / 4 * rows, 256), n), 256, 0, st>>>(a);
    else
      concat_kernel<1><<<dim3(ew_blocks(widest * rows, 256), n), 256, 0, st>>>(a);
    MC_LAUNCH_CHECK();
  }
  return 0;
}

}  // extern "C"
