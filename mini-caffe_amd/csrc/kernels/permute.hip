// N-d transpose.
//
// Any order that keeps a leading run of axes in place and swaps the two
// remaining contiguous axis groups (NCHW -> NHWC, order 0,2,3,1, is one) is a
// batch of plain 2-D transposes: those go through a 64x64 LDS tile so that both
// the reads and the writes are contiguous 256-byte rows.  Everything else falls
// to a gather with one thread per output element.
#include <cstdint>

#include "mc_common.h"
#include "mchip/kernels.h"

namespace mchip {
namespace {

constexpr int kMaxAxes = 8;

struct PermArgs {
  const float* __restrict__ x;
  float* __restrict__ y;
  long count;
  int n;
  int out_shape[kMaxAxes];
  long in_stride_of_out_axis[kMaxAxes];
};

__global__ __launch_bounds__(256) void permute_gather_kernel(const PermArgs a) {
  for (long i = blockIdx.x * 256L + threadIdx.x; i < a.count; i += gridDim.x * 256L) {
    long rem = i, src = 0;
#pragma unroll
    for (int d = kMaxAxes - 1; d >= 0; --d) {
      if (d < a.n) {
        const long q = rem / a.out_shape[d];
        src += (rem - q * a.out_shape[d]) * a.in_stride_of_out_axis[d];
        rem = q;
      }
    }
    a.y[i] = a.x[src];
  }
}

// y[b][c][r] = x[b][r][c] for R x C matrices; grid (tiles_c, tiles_r, batch).
__global__ __launch_bounds__(256) void transpose_tile_kernel(const float* __restrict__ x,
                                                             float* __restrict__ y, int R, int C) {
  __shared__ float tile[64][65];
  const long base = (long)blockIdx.z * R * C;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = r0 + ty + 4 * i, c = c0 + tx;
    if (r < R && c < C) tile[ty + 4 * i][tx] = x[base + (long)r * C + c];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int c = c0 + ty + 4 * i, r = r0 + tx;
    if (r < R && c < C) y[base + (long)c * R + r] = tile[tx][ty + 4 * i];
  }
}

// The same transpose with 16-byte accesses on both sides (R and C multiples of 4, both
// blobs 16-byte aligned): a thread loads four consecutive columns of a row, and stores
// four consecutive rows of a column.  64 x 64 tile, 256 threads, four passes each way.
__global__ __launch_bounds__(256) void transpose_tile_vec_kernel(const float* __restrict__ x,
                                                                 float* __restrict__ y, int R,
                                                                 int C) {
  __shared__ float tile[64][65];
  const long base = (long)blockIdx.z * R * C;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int quad = threadIdx.x & 15, line = threadIdx.x >> 4;  // 16 quads per tile line, 16 lines per pass
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + line + 16 * i, c = c0 + 4 * quad;
    if (r < R && c < C) {
      const float4 v = *reinterpret_cast<const float4*>(x + base + (long)r * C + c);
      float* t = &tile[line + 16 * i][4 * quad];
      t[0] = v.x;
      t[1] = v.y;
      t[2] = v.z;
      t[3] = v.w;
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = c0 + line + 16 * i, r = r0 + 4 * quad;
    if (r < R && c < C) {
      const int tc = line + 16 * i, tr = 4 * quad;
      *reinterpret_cast<float4*>(y + base + (long)c * R + r) =
          make_float4(tile[tr][tc], tile[tr + 1][tc], tile[tr + 2][tc], tile[tr + 3][tc]);
    }
  }
}

}  // namespace
}  // namespace mchip

using namespace mchip;

extern "C" int mcPermute(const float* bottom, float* top, int n, const int* shape,
                         const int* order, void* stream) {
  MC_REQUIRE(bottom && top && shape && order, "mcPermute: null argument");
  MC_REQUIRE(n >= 1 && n <= kMaxAxes, "mcPermute: 1..8 axes supported");
  MC_REQUIRE(bottom != top, "mcPermute: cannot run in place");
  long count = 1;
  bool seen[kMaxAxes] = {false};
  for (int i = 0; i < n; ++i) {
    MC_REQUIRE(order[i] >= 0 && order[i] < n && !seen[order[i]],
               "there are duplicate orders");
    seen[order[i]] = true;
    MC_REQUIRE(shape[i] >= 0, "mcPermute: negative extent");
    count *= shape[i];
  }
  if (count == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // identity -> plain copy
  bool identity = true;
  for (int i = 0; i < n; ++i) identity = identity && order[i] == i;
  if (identity) return mcCopy2D(bottom, count, top, count, count, 1, stream);
  // [0..p-1 | q..n-1 | p..q-1] -> batched 2-D transpose
  int p = 0;
  while (p < n && order[p] == p) ++p;
  const int q = order[p];
  bool two_groups = q > p;
  for (int i = 0; two_groups && i < n - q; ++i) two_groups = order[p + i] == q + i;
  for (int i = 0; two_groups && i < q - p; ++i) two_groups = order[p + (n - q) + i] == p + i;
  if (two_groups) {
    long batch = 1, R = 1, C = 1;
    for (int i = 0; i < p; ++i) batch *= shape[i];
    for (int i = p; i < q; ++i) R *= shape[i];
    for (int i = q; i < n; ++i) C *= shape[i];
    if (R < (1L << 31) && C < (1L << 31) && batch < 65536 && ceil_div(R, 64) < 65536) {
      dim3 grid(ceil_div(C, 64), ceil_div(R, 64), static_cast<unsigned>(batch));
      const bool vec = R % 4 == 0 && C % 4 == 0 &&
                       ((reinterpret_cast<uintptr_t>(bottom) | reinterpret_cast<uintptr_t>(top)) & 15u) == 0;
      if (vec)
        transpose_tile_vec_kernel<<<grid, 256, 0, st>>>(bottom, top, static_cast<int>(R),
                                                        static_cast<int>(C));
      else
        transpose_tile_kernel<<<grid, 256, 0, st>>>(bottom, top, static_cast<int>(R),
                                                    static_cast<int>(C));
      MC_LAUNCH_CHECK();
      return 0;
    }
  }
  PermArgs a;
  a.x = bottom;
  a.y = top;
  a.count = count;
  a.n = n;
  long in_stride[kMaxAxes];
  long s = 1;
  for (int i = n - 1; i >= 0; --i) {
    in_stride[i] = s;
    s *= shape[i];
  }
  for (int i = 0; i < kMaxAxes; ++i) {
    a.out_shape[i] = i < n ? shape[order[i]] : 1;
    a.in_stride_of_out_axis[i] = i < n ? in_stride[order[i]] : 0;
  }
  permute_gather_kernel<<<ew_blocks(count, 256), 256, 0, st>>>(a);
  MC_LAUNCH_CHECK();
  return 0;
}
