// The less common layers of the model zoo, each one launch and HBM-bound:
// scalar-parameter unary functions, PReLU, both LRN regions, ArgMax, Reduction,
// MVN, row gather (Embed / Filter), Crop and Tile.
//
// Layout is NCHW throughout; every kernel reads each input value once from HBM
// (window reads of LRN and the second passes of MVN hit cache) and writes each
// output once, with neighbouring threads on neighbouring addresses.
#include "mc_common.h"
#include "mchip/kernels.h"

#include <cfloat>

namespace mchip {
namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Sum over a workgroup of 256 threads; every thread gets the result.
__device__ __forceinline__ float block_sum256(float v, float* lds4) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = v;
  __syncthreads();
  return (lds4[0] + lds4[1]) + (lds4[2] + lds4[3]);
}

// ---- unary functions ----------------------------------------------------------

template <int OP>
__device__ __forceinline__ float unary(float x, float p0, float p1, float p2) {
  switch (OP) {
    case MC_UNARY_POWER: {  // (p1 + p0 * x) ^ p2
      float t = x;
      if (p0 != 1.f) t *= p0;
      if (p1 != 0.f) t += p1;
      if (p2 == 2.f) return t * t;
      if (p2 != 1.f) t = powf(t, p2);
      return t;
    }
    case MC_UNARY_EXP: {  // p1 * exp(p0 * x)
      float t = expf(p0 == 1.f ? x : p0 * x);
      return p1 == 1.f ? t : t * p1;
    }
    case MC_UNARY_LOG: {  // p2 * log(p1 + p0 * x)
      float t = x;
      if (p0 != 1.f) t *= p0;
      if (p1 != 0.f) t += p1;
      t = logf(t);
      return p2 == 1.f ? t : t * p2;
    }
    case MC_UNARY_ABS:
      return fabsf(x);
    case MC_UNARY_BNLL:  // log(1 + exp(x)), written so that exp never overflows
      return x > 0.f ? x + log1pf(expf(-x)) : log1pf(expf(x));
    case MC_UNARY_ELU:  // max(x, 0) + p0 * (exp(min(x, 0)) - 1)
      return fmaxf(x, 0.f) + p0 * (expf(fminf(x, 0.f)) - 1.f);
    case MC_UNARY_THRESHOLD:
      return x > p0 ? 1.f : 0.f;
  }
  return x;
}

// n4 float4 vectors first, then the remaining scalars.
template <int OP>
__global__ __launch_bounds__(256) void unary_kernel(const float* __restrict__ x,
                                                    float* __restrict__ y, long n, long n4,
                                                    float p0, float p1, float p2) {
  const long stride = static_cast<long>(gridDim.x) * blockDim.x;
  const long first = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x;
  const float4* __restrict__ x4 = reinterpret_cast<const float4*>(x);
  float4* __restrict__ y4 = reinterpret_cast<float4*>(y);
  for (long i = first; i < n4; i += stride) {
    float4 v = x4[i];
    v.x = unary<OP>(v.x, p0, p1, p2);
    v.y = unary<OP>(v.y, p0, p1, p2);
    v.z = unary<OP>(v.z, p0, p1, p2);
    v.w = unary<OP>(v.w, p0, p1, p2);
    y4[i] = v;
  }
  for (long i = (n4 << 2) + first; i < n; i += stride) y[i] = unary<OP>(x[i], p0, p1, p2);
}

template <int OP>
int launch_unary(const float* x, float* y, long n, float p0, float p1, float p2,
                 hipStream_t s) {
  // The float4 walk needs 16-byte aligned pointers; blobs are, offset views may not be.
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
  const long n4 = aligned ? n >> 2 : 0;
  unary_kernel<OP><<<ew_blocks(n, 256, aligned ? 4 : 1), 256, 0, s>>>(x, y, n, n4, p0, p1, p2);
  MC_LAUNCH_CHECK();
  return 0;
}

// ---- PReLU --------------------------------------------------------------------

// VEC = 4 requires inner % 4 == 0 (the four values share a channel) and 16-byte
// aligned blobs.  n < 2^32 elements, so the channel comes from 32-bit divisions.
template <int VEC>
__global__ __launch_bounds__(256) void prelu_kernel(const float* __restrict__ x,
                                                    float* __restrict__ y, long n, int channels,
                                                    int inner, const float* __restrict__ slope,
                                                    int shared) {
  const long nv = n / VEC;
  const long stride = static_cast<long>(gridDim.x) * blockDim.x;
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < nv; i += stride) {
    const unsigned e = static_cast<unsigned>(i) * VEC;
    const float sl = slope[shared ? 0u : (e / static_cast<unsigned>(inner)) % static_cast<unsigned>(channels)];
    if (VEC == 4) {
      float4 v = reinterpret_cast<const float4*>(x)[i];
      v.x = fmaxf(v.x, 0.f) + sl * fminf(v.x, 0.f);
      v.y = fmaxf(v.y, 0.f) + sl * fminf(v.y, 0.f);
      v.z = fmaxf(v.z, 0.f) + sl * fminf(v.z, 0.f);
      v.w = fmaxf(v.w, 0.f) + sl * fminf(v.w, 0.f);
      reinterpret_cast<float4*>(y)[i] = v;
    } else {
      const float v = x[i];
      y[i] = fmaxf(v, 0.f) + sl * fminf(v, 0.f);
    }
  }
}

// ---- LRN ----------------------------------------------------------------------

constexpr int kLrnChunk = 32;  // channels walked by one thread

// scale^(-beta) for a scale >= k > 0 through the hardware's base-2 logarithm and
// exponential (a few units in the last place, far inside the layer's tolerance;
// the library powf costs several times the rest of the kernel).
__device__ __forceinline__ float lrn_pow(float scale, float neg_beta) {
  return __builtin_amdgcn_exp2f(neg_beta * __builtin_amdgcn_logf(scale));
}

// One thread per (image, channel chunk, pixel): the window sum of squares is
// built directly for the chunk's first channel and then slides.
__global__ __launch_bounds__(256) void lrn_across_kernel(const float* __restrict__ x,
                                                         float* __restrict__ y, int num, int C,
                                                         int spatial, int size, float alpha_over_n,
                                                         float neg_beta, float k, int chunks) {
  const long total = static_cast<long>(num) * chunks * spatial;
  const long gid = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x;
  if (gid >= total) return;
  const int p = static_cast<int>(gid % spatial);
  const long t = gid / spatial;
  const int chunk = static_cast<int>(t % chunks);
  const int n = static_cast<int>(t / chunks);
  const int c0 = chunk * kLrnChunk;
  const int c1 = min(C, c0 + kLrnChunk);
  const int pre = (size - 1) / 2, post = size - pre - 1;
  const float* __restrict__ xi = x + (static_cast<long>(n) * C) * spatial + p;
  float* __restrict__ yi = y + (static_cast<long>(n) * C) * spatial + p;
  float acc = 0.f;
  for (int c = max(0, c0 - pre); c <= min(C - 1, c0 + post); ++c) {
    const float v = xi[static_cast<long>(c) * spatial];
    acc += v * v;
  }
  for (int c = c0; c < c1; ++c) {
    const float v = xi[static_cast<long>(c) * spatial];
    yi[static_cast<long>(c) * spatial] = v * lrn_pow(k + acc * alpha_over_n, neg_beta);
    const int head = c + 1 + post, tail = c - pre;
    if (head < C) {
      const float h = xi[static_cast<long>(head) * spatial];
      acc += h * h;
    }
    if (tail >= 0) {
      const float u = xi[static_cast<long>(tail) * spatial];
      acc -= u * u;
    }
  }
}

// The same for the usual window sizes: the chunk is walked in blocks of eight
// channels whose new values are loaded together (eight independent loads in
// flight, every value read once per thread), and each window sum is formed
// from the values in registers instead of sliding by add and subtract.
template <int SIZE>
__global__ __launch_bounds__(256) void lrn_across_fixed_kernel(const float* __restrict__ x,
                                                               float* __restrict__ y, int num, int C,
                                                               int spatial, float alpha_over_n,
                                                               float neg_beta, float k, int chunks) {
  constexpr int PRE = (SIZE - 1) / 2, B = 8;
  const long total = static_cast<long>(num) * chunks * spatial;
  const long gid = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x;
  if (gid >= total) return;
  const int p = static_cast<int>(gid % spatial);
  const long t = gid / spatial;
  const int chunk = static_cast<int>(t % chunks);
  const int n = static_cast<int>(t / chunks);
  const int c0 = chunk * kLrnChunk;
  const int c1 = min(C, c0 + kLrnChunk);
  const float* __restrict__ xi = x + (static_cast<long>(n) * C) * spatial + p;
  float* __restrict__ yi = y + (static_cast<long>(n) * C) * spatial + p;
  float win[B + SIZE - 1];  // channels cb - PRE .. cb + B - 1 + PRE of the current block
#pragma unroll
  for (int i = 0; i < SIZE - 1; ++i) {
    const int c = c0 - PRE + i;
    win[i] = (c >= 0 && c < C) ? xi[static_cast<long>(c) * spatial] : 0.f;
  }
  for (int cb = c0; cb < c1; cb += B) {
#pragma unroll
    for (int j = 0; j < B; ++j) {
      const int c = cb + PRE + j;
      win[SIZE - 1 + j] = c < C ? xi[static_cast<long>(c) * spatial] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < B; ++j) {
      if (cb + j < c1) {
        float acc = 0.f;
#pragma unroll
        for (int d = 0; d < SIZE; ++d) acc += win[j + d] * win[j + d];
        yi[static_cast<long>(cb + j) * spatial] = win[j + PRE] * lrn_pow(k + acc * alpha_over_n, neg_beta);
      }
    }
#pragma unroll
    for (int i = 0; i < SIZE - 1; ++i) win[i] = win[B + i];
  }
}

// One thread per element: the padded-average of squares over a size x size
// window (divisor counts the padding, as the average pooling it stands for).
__global__ __launch_bounds__(256) void lrn_within_kernel(const float* __restrict__ x,
                                                         float* __restrict__ y, long planes, int H,
                                                         int W, int size, float alpha,
                                                         float neg_beta) {
  const long total = planes * H * W;
  const long gid = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x;
  if (gid >= total) return;
  const int w = static_cast<int>(gid % W);
  const int h = static_cast<int>((gid / W) % H);
  const float* __restrict__ xp = x + (gid / (static_cast<long>(H) * W)) * H * W;
  const int pad = (size - 1) / 2;
  int hs = h - pad, ws = w - pad;
  int he = min(hs + size, H + pad), we = min(ws + size, W + pad);
  const float pool = static_cast<float>((he - hs) * (we - ws));
  hs = max(hs, 0);
  ws = max(ws, 0);
  he = min(he, H);
  we = min(we, W);
  float acc = 0.f;
  for (int i = hs; i < he; ++i)
    for (int j = ws; j < we; ++j) {
      const float v = xp[i * W + j];
      acc += v * v;
    }
  y[gid] = x[gid] * lrn_pow(1.f + alpha * (acc / pool), neg_beta);
}

// ---- ArgMax -------------------------------------------------------------------

// Order of the reference's std::greater on (value, index) pairs: larger value
// first, and among equal values the larger index first.
__device__ __forceinline__ bool pair_after(float v, int i, float bv, int bi) {
  return v > bv || (v == bv && i > bi);
}

__device__ __forceinline__ void store_argmax(float* __restrict__ y, long o, int in, int inner,
                                             int top_k, int j, int layout, float v, int idx) {
  if (layout == MC_ARGMAX_INDEX)
    y[(o * top_k + j) * inner + in] = static_cast<float>(idx);
  else if (layout == MC_ARGMAX_VALUE)
    y[(o * top_k + j) * inner + in] = v;
  else {  // MC_ARGMAX_INDEX_THEN_VALUE, inner == 1
    y[2 * o * top_k + j] = static_cast<float>(idx);
    y[2 * o * top_k + top_k + j] = v;
  }
}

// One thread per (outer, inner) line: top_k selection passes over dim values.
__global__ __launch_bounds__(256) void argmax_thread_kernel(const float* __restrict__ x,
                                                            float* __restrict__ y, long lines,
                                                            int dim, int inner, int top_k,
                                                            int layout) {
  const long gid = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x;
  if (gid >= lines) return;
  const long o = gid / inner;
  const int in = static_cast<int>(gid % inner);
  const float* __restrict__ xl = x + o * dim * inner + in;
  float pv = 0.f;
  int pi = -1;
  for (int j = 0; j < top_k; ++j) {
    float bv = 0.f;
    int bi = -1;
    for (int d = 0; d < dim; ++d) {
      const float v = xl[static_cast<long>(d) * inner];
      if (pi >= 0 && !pair_after(pv, pi, v, d)) continue;  // already emitted
      if (bi < 0 || pair_after(v, d, bv, bi)) {
        bv = v;
        bi = d;
      }
    }
    store_argmax(y, o, in, inner, top_k, j, layout, bv, bi);
    pv = bv;
    pi = bi;
  }
}

// One workgroup per line, for long lines.
__global__ __launch_bounds__(256) void argmax_block_kernel(const float* __restrict__ x,
                                                           float* __restrict__ y, int dim,
                                                           int inner, int top_k, int layout) {
  __shared__ float s_v[4];
  __shared__ int s_i[4];
  const long line = blockIdx.x;
  const long o = line / inner;
  const int in = static_cast<int>(line % inner);
  const float* __restrict__ xl = x + o * dim * inner + in;
  float pv = 0.f;
  int pi = -1;
  for (int j = 0; j < top_k; ++j) {
    float bv = 0.f;
    int bi = -1;
    for (int d = threadIdx.x; d < dim; d += 256) {
      const float v = xl[static_cast<long>(d) * inner];
      if (pi >= 0 && !pair_after(pv, pi, v, d)) continue;
      if (bi < 0 || pair_after(v, d, bv, bi)) {
        bv = v;
        bi = d;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (oi >= 0 && (bi < 0 || pair_after(ov, oi, bv, bi))) {
        bv = ov;
        bi = oi;
      }
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) {
      s_v[threadIdx.x >> 6] = bv;
      s_i[threadIdx.x >> 6] = bi;
    }
    __syncthreads();
    bv = s_v[0];
    bi = s_i[0];
#pragma unroll
    for (int w = 1; w < 4; ++w)
      if (s_i[w] >= 0 && (bi < 0 || pair_after(s_v[w], s_i[w], bv, bi))) {
        bv = s_v[w];
        bi = s_i[w];
      }
    if (threadIdx.x == 0) store_argmax(y, o, in, inner, top_k, j, layout, bv, bi);
    pv = bv;
    pi = bi;
  }
}

// ---- Reduction ----------------------------------------------------------------

__device__ __forceinline__ float reduce_term(int op, float v) {
  return op == MC_REDUCE_ASUM ? fabsf(v) : (op == MC_REDUCE_SUMSQ ? v * v : v);
}

__global__ __launch_bounds__(256) void reduction_block_kernel(int op, const float* __restrict__ x,
                                                              float* __restrict__ y, int dim,
                                                              float coeff) {
  __shared__ float red[4];
  const float* __restrict__ xr = x + static_cast<long>(blockIdx.x) * dim;
  float acc = 0.f;
  for (int d = threadIdx.x; d < dim; d += 256) acc += reduce_term(op, xr[d]);
  acc = block_sum256(acc, red);
  if (threadIdx.x == 0) y[blockIdx.x] = acc * coeff;
}

__global__ __launch_bounds__(256) void reduction_thread_kernel(int op, const float* __restrict__ x,
                                                               float* __restrict__ y, int num,
                                                               int dim, float coeff) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= num) return;
  const float* __restrict__ xr = x + static_cast<long>(r) * dim;
  float acc = 0.f;
  for (int d = 0; d < dim; ++d) acc += reduce_term(op, xr[d]);
  y[r] = acc * coeff;
}

// ---- MVN ----------------------------------------------------------------------

__global__ __launch_bounds__(256) void mvn_kernel(const float* __restrict__ x,
                                                  float* __restrict__ y, int dim, int normalize,
                                                  float eps) {
  __shared__ float red[4];
  const float* __restrict__ xr = x + static_cast<long>(blockIdx.x) * dim;
  float* __restrict__ yr = y + static_cast<long>(blockIdx.x) * dim;
  const float inv = 1.f / static_cast<float>(dim);
  float s = 0.f;
  for (int d = threadIdx.x; d < dim; d += 256) s += xr[d];
  const float mean = block_sum256(s, red) * inv;
  float div = 1.f;
  if (normalize) {
    float q = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) {
      const float t = xr[d] - mean;
      q += t * t;
    }
    div = sqrtf(block_sum256(q, red) * inv) + eps;
  }
  for (int d = threadIdx.x; d < dim; d += 256) {
    const float t = xr[d] - mean;
    yr[d] = normalize ? t / div : t;
  }
}

// ---- row gather, crop, tile ---------------------------------------------------

__global__ __launch_bounds__(256) void gather_rows_kernel(const float* __restrict__ table,
                                                          const float* __restrict__ rows,
                                                          const float* __restrict__ bias,
                                                          float* __restrict__ y, long total,
                                                          int row_len, int table_rows) {
  const long stride = static_cast<long>(gridDim.x) * blockDim.x;
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < total; i += stride) {
    const long r = i / row_len;
    const int j = static_cast<int>(i - r * row_len);
    const int src = static_cast<int>(rows[r]);
    float v = src >= 0 && src < table_rows ? table[static_cast<long>(src) * row_len + j]
                                           : __int_as_float(0x7fc00000);
    if (bias) v += bias[j];
    y[i] = v;
  }
}

struct CropArgs {
  int num_axes;
  int top_shape[MC_MAX_AXES];
  long bottom_stride[MC_MAX_AXES];
  long base;  // offset of the crop's origin in the bottom blob
};

__global__ __launch_bounds__(256) void crop_kernel(const float* __restrict__ x,
                                                   float* __restrict__ y, long total, CropArgs a) {
  const long stride = static_cast<long>(gridDim.x) * blockDim.x;
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < total; i += stride) {
    long rest = i, src = a.base;
    for (int ax = a.num_axes - 1; ax >= 0; --ax) {
      const long q = rest / a.top_shape[ax];
      src += (rest - q * a.top_shape[ax]) * a.bottom_stride[ax];
      rest = q;
    }
    y[i] = x[src];
  }
}

__global__ __launch_bounds__(256) void tile_kernel(const float* __restrict__ x,
                                                   float* __restrict__ y, long total, int inner,
                                                   int tiles) {
  const long stride = static_cast<long>(gridDim.x) * blockDim.x;
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < total; i += stride) {
    const long q = i / inner;  // = outer index * tiles + tile
    y[i] = x[(q / tiles) * inner + (i - q * inner)];
  }
}

}  // namespace
}  // namespace mchip

using namespace mchip;

extern "C" {

int mcUnary(int op, const float* bottom, float* top, long count, float p0, float p1, float p2,
            void* stream) {
  MC_REQUIRE(count >= 0, "mcUnary: negative count");
  if (count == 0) return 0;
  MC_REQUIRE(bottom && top, "mcUnary: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (op) {
    case MC_UNARY_POWER: return launch_unary<MC_UNARY_POWER>(bottom, top, count, p0, p1, p2, s);
    case MC_UNARY_EXP: return launch_unary<MC_UNARY_EXP>(bottom, top, count, p0, p1, p2, s);
    case MC_UNARY_LOG: return launch_unary<MC_UNARY_LOG>(bottom, top, count, p0, p1, p2, s);
    case MC_UNARY_ABS: return launch_unary<MC_UNARY_ABS>(bottom, top, count, p0, p1, p2, s);
    case MC_UNARY_BNLL: return launch_unary<MC_UNARY_BNLL>(bottom, top, count, p0, p1, p2, s);
    case MC_UNARY_ELU: return launch_unary<MC_UNARY_ELU>(bottom, top, count, p0, p1, p2, s);
    case MC_UNARY_THRESHOLD:
      return launch_unary<MC_UNARY_THRESHOLD>(bottom, top, count, p0, p1, p2, s);
  }
  return fail("mcUnary: unknown op %d", op);
}

int mcPReLU(const float* bottom, float* top, int outer, int channels, int inner,
            const float* slope, int channel_shared, void* stream) {
  MC_REQUIRE(outer >= 0 && channels > 0 && inner > 0, "mcPReLU: bad extents %d x %d x %d", outer,
             channels, inner);
  const long n = static_cast<long>(outer) * channels * inner;
  if (n == 0) return 0;
  MC_REQUIRE(bottom && top && slope, "mcPReLU: null pointer");
  MC_REQUIRE(n < (1L << 32), "mcPReLU: blob too large");
  const bool vec = inner % 4 == 0 && (reinterpret_cast<uintptr_t>(bottom) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(top) & 15) == 0;
  if (vec)
    prelu_kernel<4><<<ew_blocks(n / 4, 256), 256, 0, static_cast<hipStream_t>(stream)>>>(
        bottom, top, n, channels, inner, slope, channel_shared);
  else
    prelu_kernel<1><<<ew_blocks(n, 256, 4), 256, 0, static_cast<hipStream_t>(stream)>>>(
        bottom, top, n, channels, inner, slope, channel_shared);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcLRNAcrossChannels(const float* bottom, float* top, int num, int channels, int height,
                        int width, int local_size, float alpha, float beta, float k,
                        void* stream) {
  MC_REQUIRE(num >= 0 && channels > 0 && height > 0 && width > 0, "mcLRNAcrossChannels: bad shape");
  MC_REQUIRE(local_size > 0 && (local_size & 1), "LRN only supports odd values for local_size");
  if (num == 0) return 0;
  MC_REQUIRE(bottom && top && bottom != top, "mcLRNAcrossChannels: null or aliased pointers");
  const int spatial = height * width;
  const int chunks = ceil_div(channels, kLrnChunk);
  const long total = static_cast<long>(num) * chunks * spatial;
  MC_REQUIRE(total < (1L << 31) * 256, "mcLRNAcrossChannels: blob too large");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int blocks = ceil_div(total, 256);
  const float an = alpha / local_size;
  if (local_size == 3)
    lrn_across_fixed_kernel<3><<<blocks, 256, 0, st>>>(bottom, top, num, channels, spatial, an, -beta, k, chunks);
  else if (local_size == 5)
    lrn_across_fixed_kernel<5><<<blocks, 256, 0, st>>>(bottom, top, num, channels, spatial, an, -beta, k, chunks);
  else if (local_size == 7)
    lrn_across_fixed_kernel<7><<<blocks, 256, 0, st>>>(bottom, top, num, channels, spatial, an, -beta, k, chunks);
  else
    lrn_across_kernel<<<blocks, 256, 0, st>>>(bottom, top, num, channels, spatial, local_size, an, -beta, k,
                                              chunks);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcLRNWithinChannel(const float* bottom, float* top, long planes, int height, int width,
                       int local_size, float alpha, float beta, void* stream) {
  MC_REQUIRE(planes >= 0 && height > 0 && width > 0, "mcLRNWithinChannel: bad shape");
  MC_REQUIRE(local_size > 0 && (local_size & 1), "LRN only supports odd values for local_size");
  if (planes == 0) return 0;
  MC_REQUIRE(bottom && top && bottom != top, "mcLRNWithinChannel: null or aliased pointers");
  const long total = planes * height * width;
  MC_REQUIRE(total < (1L << 31) * 256, "mcLRNWithinChannel: blob too large");
  lrn_within_kernel<<<ceil_div(total, 256), 256, 0, static_cast<hipStream_t>(stream)>>>(
      bottom, top, planes, height, width, local_size, alpha, -beta);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcArgMax(const float* bottom, float* top, long outer, int dim, int inner, int top_k,
             int layout, void* stream) {
  MC_REQUIRE(outer >= 0 && dim > 0 && inner > 0, "mcArgMax: bad extents");
  MC_REQUIRE(top_k >= 1 && top_k <= dim, "mcArgMax: top_k %d outside [1, %d]", top_k, dim);
  MC_REQUIRE(layout == MC_ARGMAX_INDEX || layout == MC_ARGMAX_VALUE ||
                 (layout == MC_ARGMAX_INDEX_THEN_VALUE && inner == 1),
             "mcArgMax: layout %d not valid for inner = %d", layout, inner);
  MC_REQUIRE(dim < (1 << 24), "mcArgMax: indices above 2^24 are not exact in float");
  const long lines = outer * inner;
  if (lines == 0) return 0;
  MC_REQUIRE(bottom && top && bottom != top, "mcArgMax: null or aliased pointers");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool per_thread = lines >= 8192 && static_cast<long>(dim) * top_k <= 8192;
  if (per_thread || dim <= 64) {
    argmax_thread_kernel<<<ceil_div(lines, 256), 256, 0, s>>>(bottom, top, lines, dim, inner,
                                                               top_k, layout);
  } else {
    MC_REQUIRE(lines < (1L << 31), "mcArgMax: too many lines");
    argmax_block_kernel<<<static_cast<int>(lines), 256, 0, s>>>(bottom, top, dim, inner, top_k,
                                                                 layout);
  }
  MC_LAUNCH_CHECK();
  return 0;
}

int mcReduction(int op, const float* bottom, float* top, int num, int dim, float coeff,
                void* stream) {
  MC_REQUIRE(op >= MC_REDUCE_SUM && op <= MC_REDUCE_MEAN, "Unknown reduction op: %d", op);
  MC_REQUIRE(num >= 0 && dim > 0, "mcReduction: bad extents %d x %d", num, dim);
  if (num == 0) return 0;
  MC_REQUIRE(bottom && top, "mcReduction: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (op == MC_REDUCE_MEAN) coeff /= static_cast<float>(dim);
  if (dim <= 64 && num >= 1024)
    reduction_thread_kernel<<<ceil_div(num, 256), 256, 0, s>>>(op, bottom, top, num, dim, coeff);
  else
    reduction_block_kernel<<<num, 256, 0, s>>>(op, bottom, top, dim, coeff);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcMVN(const float* bottom, float* top, int num, int dim, int normalize_variance, float eps,
          void* stream) {
  MC_REQUIRE(num >= 0 && dim > 0, "mcMVN: bad extents %d x %d", num, dim);
  if (num == 0) return 0;
  MC_REQUIRE(bottom && top, "mcMVN: null pointer");
  mvn_kernel<<<num, 256, 0, static_cast<hipStream_t>(stream)>>>(bottom, top, dim,
                                                               normalize_variance, eps);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcGatherRows(const float* table, int table_rows, int row_len, const float* rows, long num_rows,
                 const float* bias, float* top, void* stream) {
  MC_REQUIRE(table_rows > 0 && row_len > 0 && num_rows >= 0, "mcGatherRows: bad extents");
  MC_REQUIRE(table_rows < (1 << 24), "mcGatherRows: row numbers above 2^24 are not exact in float");
  if (num_rows == 0) return 0;
  MC_REQUIRE(table && rows && top, "mcGatherRows: null pointer");
  const long total = num_rows * row_len;
  gather_rows_kernel<<<ew_blocks(total, 256, 4), 256, 0, static_cast<hipStream_t>(stream)>>>(
      table, rows, bias, top, total, row_len, table_rows);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcCrop(const float* bottom, float* top, int num_axes, const int* bottom_shape,
           const int* top_shape, const int* offsets, void* stream) {
  MC_REQUIRE(num_axes >= 1 && num_axes <= MC_MAX_AXES, "mcCrop: %d axes (1..%d supported)",
             num_axes, MC_MAX_AXES);
  CropArgs a;
  a.num_axes = num_axes;
  a.base = 0;
  long total = 1, stride = 1;
  for (int ax = num_axes - 1; ax >= 0; --ax) {
    MC_REQUIRE(offsets[ax] >= 0 && top_shape[ax] >= 0 &&
                   bottom_shape[ax] - offsets[ax] >= top_shape[ax],
               "the crop for dimension %d is out-of-bounds with size %d and offset %d", ax,
               top_shape[ax], offsets[ax]);
    a.top_shape[ax] = top_shape[ax];
    a.bottom_stride[ax] = stride;
    a.base += offsets[ax] * stride;
    stride *= bottom_shape[ax];
    total *= top_shape[ax];
  }
  if (total == 0) return 0;
  MC_REQUIRE(bottom && top, "mcCrop: null pointer");
  crop_kernel<<<ew_blocks(total, 256, 4), 256, 0, static_cast<hipStream_t>(stream)>>>(bottom, top,
                                                                                      total, a);
  MC_LAUNCH_CHECK();
  return 0;
}

int mcTile(const float* bottom, float* top, long outer, int inner, int tiles, void* stream) {
  MC_REQUIRE(outer >= 0 && inner > 0 && tiles > 0, "Number of tiles must be positive.");
  const long total = outer * tiles * inner;
  if (total == 0) return 0;
  MC_REQUIRE(bottom && top && bottom != top, "mcTile: null or aliased pointers");
  tile_kernel<<<ew_blocks(total, 256, 4), 256, 0, static_cast<hipStream_t>(stream)>>>(
      bottom, top, total, inner, tiles);
  MC_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
