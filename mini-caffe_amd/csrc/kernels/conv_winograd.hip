// 3x3 stride-1 convolution through the Winograd minimal-filtering identity
// F(2x2, 3x3): a 2x2 block of outputs of one channel pair needs 16 products
// instead of 36,
//
//     Y = A^T [ (G g G^T) .* (B^T d B) ] A,
//
// d the 4x4 input patch under the block, g the 3x3 filter.  Summed over the
// input channels the element-wise products are sixteen independent matrix
// products  M_f[Cout][T] = U_f[Cout][Cin] * V_f[Cin][T]  (f = position in the
// 4x4 transform, T = 2x2 output blocks of the whole batch).  One kernel does all
// of it for a tile of 64 output channels x 32 blocks:
//
//   loader    every thread fetches three rows of a block's 4x4 patch of one
//             channel straight from the bottom blob, forms eight of the sixteen
//             V values in registers and stores them as the B operands in LDS;
//             the transformed filters U (packed once per weight change in the
//             order the tile consumes them) are copied to LDS as they are;
//   products  wavefront w multiplies the four transform positions of row w,
//             f = 4 w .. 4 w + 3: 8 accumulator blocks of 32 x 32 per wavefront,
//             v_mfma_f32_32x32x2_f32;
//   finish    A^T m A: the sums over a transform row in registers, the sums
//             over the four rows (= wavefronts) through LDS, then the layer's
//             epilogue (scale, shift, residual, activation) and the store.
//
// Neither V nor M ever exists in memory: the launch reads the bottom blob and
// the filters and writes the top blob.  Replaces the same reference code as the
// direct path (conv_layer.cu:7-22 with base_conv_layer.cpp:254-278); sums are
// associated differently from a direct convolution (transformed operands, K
// order over input channels only), within the usual fp32 rounding of either.
#include "conv_internal.h"
#include "mc_common.h"
#include "mchip/kernels.h"

#include <algorithm>

namespace mchip {

namespace {

constexpr int kTileM = 64;   // output channels of a tile
constexpr int kTileT = 32;   // 2x2 output blocks of a tile
constexpr int kStageC = 4;   // input channels per K stage
constexpr int kAStage = 16 * kTileM * kStageC;  // floats of U per stage and tile
constexpr int kBStage = 16 * kTileT * kStageC;  // floats of V per stage and tile
constexpr int kBufferFlags = 0x00020000;        // raw dword buffer, offsets range-checked
constexpr unsigned kNoElement = 0x80000000u;    // beyond every buffer this file builds

typedef float acc16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

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

// Transformed filters in the order a tile's stages read them:
//   u[mt][kt][f][kp][m][e] = (G g G^T)[f / 4][f % 4]  of filter (co, ci),
//   co = 64 mt + m, ci = 4 kt + 2 kp + e,  G = [1 0 0; 1/2 1/2 1/2; 1/2 -1/2 1/2; 0 0 1],
// zero where co or ci lie past the layer's channels (KT is even: the loader works in
// rounds of eight channels).  One thread per (co, ci) of the padded extents.
__global__ __launch_bounds__(256) void winograd_pack_filter_kernel(const float* __restrict__ w,
                                                                   float* __restrict__ u, int Cout,
                                                                   int C, int MT, int KT) {
  const long i = blockIdx.x * 256L + threadIdx.x;
  const int cpad = KT * kStageC;
  if (i >= (long)MT * kTileM * cpad) return;
  const int co = static_cast<int>(i / cpad), ci = static_cast<int>(i % cpad);
  float g[3][3];
#pragma unroll
  for (int r = 0; r < 3; ++r)
#pragma unroll
    for (int c = 0; c < 3; ++c)
      g[r][c] = (co < Cout && ci < C) ? w[((long)co * C + ci) * 9 + r * 3 + c] : 0.f;
  float t[4][3];
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    t[0][c] = g[0][c];
    t[1][c] = 0.5f * (g[0][c] + g[1][c] + g[2][c]);
    t[2][c] = 0.5f * (g[0][c] - g[1][c] + g[2][c]);
    t[3][c] = g[2][c];
  }
  const int mt = co / kTileM, m = co % kTileM;
  const int kt = ci / kStageC, kp = (ci % kStageC) / 2, e = ci % 2;
  float* out = u + ((long)mt * KT + kt) * kAStage + kp * (kTileM * 2) + m * 2 + e;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    out[(r * 4 + 0) * (kTileM * kStageC)] = t[r][0];
    out[(r * 4 + 1) * (kTileM * kStageC)] = 0.5f * (t[r][0] + t[r][1] + t[r][2]);
    out[(r * 4 + 2) * (kTileM * kStageC)] = 0.5f * (t[r][0] - t[r][1] + t[r][2]);
    out[(r * 4 + 3) * (kTileM * kStageC)] = t[r][2];
  }
}

struct WinogradArgs {
  const float* __restrict__ x;   // bottom [num, C, H, W]
  const float* __restrict__ u;   // packed filters, see winograd_pack_filter_kernel
  float* __restrict__ y;         // top [num, c_first, Ho, Wo]
  float* __restrict__ y_second;  // [num, Cout - c_first, Ho, Wo] or null
  const float* __restrict__ scale;
  const float* __restrict__ shift;
  const float* __restrict__ residual;
  unsigned x_bytes, u_bytes;
  int C, H, W, HW;
  int x_nstride;  // C * H * W
  int Cout, Ho, Wo, HoWo;
  int pad_h, pad_w;
  int Tw, ThTw, T;  // blocks across, per image, in the run
  unsigned div_img_mul, div_img_shift;  // t / ThTw
  unsigned div_tw_mul, div_tw_shift;    // rem / Tw
  unsigned div_mt_mul, div_mt_shift;    // logical tile / MT
  int MT, NT, KT;
  int c_first;
  int act;
  float slope;
  int pairs;  // a block's two outputs of a row may go out as one 8-byte store
  // The channel rounds cut into slices (blockIdx.y), summed inside the launch: every
  // workgroup leaves its 64 row sums per thread in `partial`
  // ([slice][tile][value][thread]) and counts in counters[tile]; the last one to arrive
  // adds the slices in slice order, finishes the tile and puts the counter back to zero.
  int rounds_per_slice;
  float* partial;
  int* counters;
};

// Lane l of v_mfma_f32_32x32x2_f32 supplies A[l % 32][l / 32] and B[l / 32][l % 32];
// which two physical K rows form a step is free as long as both operands agree,
// so half-wave h reads the stage's channels 2 h and 2 h + 1 with one 8-byte LDS read
// and step e multiplies channels {e, 2 + e}.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void winograd_fused_kernel(
    const WinogradArgs a) {
  // K loop: As[2][f 16][kp 2][m 64][e 2], Bs[2][2][f 16][kp 2][t 32][e 2]  (64 KB);
  // finish: Es[dj 2][i 4][co 64][t 32]                                     (64 KB)
  __shared__ __attribute__((aligned(16))) float lds[2 * 4 * kTileM * kTileT];
  float* const As = lds;
  float* const Bs = lds + 2 * kAStage;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int lhi = lane >> 5;

  // Workgroup ids are dealt round-robin to the 8 XCDs: give each XCD a contiguous
  // run of logical tiles (channel tiles fastest), so the tiles that share a patch
  // tile and neighbouring patch tiles meet in one L2.
  int mt, nt;
  {
    const int total = a.MT * a.NT;
    const int bid = blockIdx.x;
    const int q = total / kNumXcd, r = total % kNumXcd;
    const int xcd = bid % kNumXcd, local = bid / kNumXcd;
    const int logical = xcd * q + (xcd < r ? xcd : r) + local;
    nt = fast_div(logical, a.div_mt_mul, a.div_mt_shift);
    mt = logical - nt * a.MT;
  }

  const __amdgpu_buffer_rsrc_t xres =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.x), 0, a.x_bytes, kBufferFlags);
  const __amdgpu_buffer_rsrc_t ures =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.u), 0, a.u_bytes, kBufferFlags);

  // Loader of the bottom blob: a round covers eight channels (two K stages).
  // Wavefront w takes channels 2 w and 2 w + 1 of the round (lane / 32), lane % 32 is
  // the block; a thread fetches the block's whole 4x4 patch of its channel with
  // sixteen dword loads whose byte offsets are fixed over the K loop (the round's
  // first channel rides in the scalar offset), forms the sixteen V values in
  // registers and stores them where the products read them.  An element outside the
  // map or past the last block has bit 31 set, which is beyond the buffer: it reads
  // as zero.  The loads of round s + 1 are issued before the products of round s and
  // first touched after them: two K stages to cover the latency of memory.
  unsigned boff[4][4];
  {
    const int t = nt * kTileT + l32;
    const bool tv = t < a.T;
    const int n = fast_div(t, a.div_img_mul, a.div_img_shift);
    const int rem = t - n * a.ThTw;
    const int ty = fast_div(rem, a.div_tw_mul, a.div_tw_shift);
    const int tx = rem - ty * a.Tw;
    const int h0 = 2 * ty - a.pad_h, w0 = 2 * tx - a.pad_w;
    const unsigned origin =
        (static_cast<unsigned>(n) * a.x_nstride + static_cast<unsigned>(2 * wave + lhi) * a.HW) * 4u;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int hh = h0 + i;
      const bool row_ok = tv && static_cast<unsigned>(hh) < static_cast<unsigned>(a.H);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int ww = w0 + j;
        const bool ok = row_ok && static_cast<unsigned>(ww) < static_cast<unsigned>(a.W);
        boff[i][j] = ok ? origin + static_cast<unsigned>(hh * a.W + ww) * 4u : kNoElement;
      }
    }
  }
  const int rounds = a.KT / 2;
  const int s_begin = blockIdx.y * a.rounds_per_slice;  // this slice's rounds (never empty)
  const int s_end = min(rounds, s_begin + a.rounds_per_slice);
  // the last round of a channel count that is no multiple of eight: a lane whose
  // channel does not exist gets the "no element" offsets before that round is fetched
  const bool ragged = (a.C & 7) != 0;
  const bool no_channel = 8 * (rounds - 1) + 2 * wave + lhi >= a.C;
#define MC_DROP_MISSING_CHANNELS()                                           \
  _Pragma("unroll") for (int i = 0; i < 4; ++i) {                            \
    _Pragma("unroll") for (int j = 0; j < 4; ++j)                            \
      boff[i][j] = no_channel ? kNoElement : boff[i][j];                     \
  }
  // LDS places (in floats) of what this thread stores and reads
  const int a_st = tid * 4;
  // (the two B buffers alternate by round: both places flip by the size of one)
  int b_st = (wave >> 1) * kBStage + (wave & 1) * (kTileT * 2) + l32 * 2 + lhi;
  const int a_rd = wave * 4 * (kTileM * kStageC) + lhi * (kTileM * 2) + l32 * 2;
  int b_rd = wave * 4 * (kTileT * kStageC) + lhi * (kTileT * 2) + l32 * 2;
  const unsigned a_voff = static_cast<unsigned>(tid) * 16u;
  const unsigned round_bytes = static_cast<unsigned>(a.HW) * 32u;  // eight channels

  float4 areg[4];
  float ereg[4][4];

#define MC_LOADF(res, voff, soff) \
  __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(res, voff, soff, 0))
#define MC_LOAD_A(kt)                                                                           \
  {                                                                                             \
    const unsigned a_soff = static_cast<unsigned>((mt * a.KT + (kt)) * kAStage) * 4u;           \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                             \
      const u32x4 w4 = __builtin_amdgcn_raw_buffer_load_b128(ures, a_voff, a_soff + i * 4096u, 0); \
      areg[i] = __builtin_bit_cast(float4, w4);                                                 \
    }                                                                                           \
  }
#define MC_LOAD_B(s)                                                                            \
  {                                                                                             \
    const unsigned b_soff = static_cast<unsigned>(s) * round_bytes;                             \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                             \
      _Pragma("unroll") for (int j = 0; j < 4; ++j) ereg[i][j] = MC_LOADF(xres, boff[i][j], b_soff); \
    }                                                                                           \
  }
#define MC_STORE_A(buf)                                                                         \
  {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < 4; ++i)                                               \
      *reinterpret_cast<float4*>(As + (buf)*kAStage + a_st + i * 1024) = areg[i];               \
  }
  // V = B^T d B, B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1]
#define MC_STORE_B()                                                                            \
  {                                                                                             \
    float* bw = Bs + (b_st ^ (2 * kBStage));                                                    \
    _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                             \
      const float r0 = ereg[0][j] - ereg[2][j], r1 = ereg[1][j] + ereg[2][j];                   \
      const float r2 = ereg[2][j] - ereg[1][j], r3 = ereg[1][j] - ereg[3][j];                   \
      ereg[0][j] = r0;                                                                          \
      ereg[1][j] = r1;                                                                          \
      ereg[2][j] = r2;                                                                          \
      ereg[3][j] = r3;                                                                          \
    }                                                                                           \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                             \
      bw[(i * 4 + 0) * (kTileT * kStageC)] = ereg[i][0] - ereg[i][2];                           \
      bw[(i * 4 + 1) * (kTileT * kStageC)] = ereg[i][1] + ereg[i][2];                           \
      bw[(i * 4 + 2) * (kTileT * kStageC)] = ereg[i][2] - ereg[i][1];                           \
      bw[(i * 4 + 3) * (kTileT * kStageC)] = ereg[i][1] - ereg[i][3];                           \
    }                                                                                           \
  }
#define MC_COMPUTE(abuf, sub)                                                             \
  {                                                                                             \
    f32x2 av[4][2], bv[4];                                                                      \
    _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                             \
      _Pragma("unroll") for (int mb = 0; mb < 2; ++mb) av[j][mb] = *reinterpret_cast<const f32x2*>( \
          As + (abuf)*kAStage + a_rd + j * (kTileM * kStageC) + mb * 64);                       \
      bv[j] = *reinterpret_cast<const f32x2*>(Bs + b_rd + (sub)*kBStage + j * (kTileT * kStageC)); \
    }                                                                                           \
    _Pragma("unroll") for (int e = 0; e < 2; ++e) {                                             \
      _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                           \
        _Pragma("unroll") for (int mb = 0; mb < 2; ++mb)                                        \
          acc[j][mb] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j][mb][e], bv[j][e], acc[j][mb], 0, 0, 0); \
      }                                                                                         \
    }                                                                                           \
  }
  // Order of a stage's instructions inside a wavefront.  A wavefront issues in order, and
  // a global load can wait for room in the memory pipeline: twenty loads at the head of
  // a stage keep the wavefront from feeding the matrix pipe for as long.  So every
  // product is followed by one or two loads (first stage of a round: the filters of
  // the second stage, then the patches of the next round) or by a share of the
  // transform and of the LDS stores (second stage), whose issue then hides under the
  // product's 64 cycles.
#define MC_SG(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define MC_ORDER_FIRST()                                                                     \
  MC_SG(0x100, 6);                                                                           \
  MC_SG(0x008, 1); MC_SG(0x020, 2); MC_SG(0x008, 1); MC_SG(0x020, 2);                        \
  MC_SG(0x008, 1); MC_SG(0x020, 2); MC_SG(0x008, 1); MC_SG(0x020, 2);                        \
  MC_SG(0x008, 1); MC_SG(0x020, 2); MC_SG(0x008, 1); MC_SG(0x020, 2);                        \
  MC_SG(0x008, 1); MC_SG(0x020, 2); MC_SG(0x008, 1); MC_SG(0x020, 2);                        \
  MC_SG(0x008, 1); MC_SG(0x020, 1); MC_SG(0x008, 1); MC_SG(0x020, 1);                        \
  MC_SG(0x008, 1); MC_SG(0x020, 1); MC_SG(0x008, 1); MC_SG(0x020, 1);                        \
  MC_SG(0x008, 1); MC_SG(0x200, 1); MC_SG(0x008, 1); MC_SG(0x200, 1);                        \
  MC_SG(0x008, 1); MC_SG(0x200, 1); MC_SG(0x008, 1); MC_SG(0x200, 1)
#define MC_ORDER_SECOND()                                                                    \
  MC_SG(0x100, 6);                                                                           \
  MC_SG(0x008, 1); MC_SG(0x020, 1); MC_SG(0x008, 1); MC_SG(0x020, 1);                        \
  MC_SG(0x008, 1); MC_SG(0x020, 1); MC_SG(0x008, 1); MC_SG(0x020, 1);                        \
  MC_SG(0x008, 1); MC_SG(0x002, 4); MC_SG(0x008, 1); MC_SG(0x002, 4);                        \
  MC_SG(0x008, 1); MC_SG(0x002, 4); MC_SG(0x008, 1); MC_SG(0x002, 4);                        \
  MC_SG(0x008, 1); MC_SG(0x002, 4); MC_SG(0x008, 1); MC_SG(0x002, 4);                        \
  MC_SG(0x008, 1); MC_SG(0x002, 4); MC_SG(0x008, 1); MC_SG(0x002, 4);                        \
  MC_SG(0x008, 1); MC_SG(0x200, 4); MC_SG(0x008, 1); MC_SG(0x200, 4);                        \
  MC_SG(0x008, 1); MC_SG(0x200, 2); MC_SG(0x008, 1); MC_SG(0x200, 2)
  // Round s: its V sits in the B buffer b_rd points into (both halves), the filters of
  // its first stage in A buffer 0.  Every round fetches what the next one needs; the
  // last round fetches its own operands once more (nobody reads them), so all rounds
  // are the same code.
#define MC_ROUND(s)                                                      \
  {                                                                      \
    const int s_next = min((s) + 1, rounds - 1);                         \
    MC_LOAD_A(2 * (s) + 1);                                              \
    MC_LOAD_B(s_next);                                                   \
    MC_COMPUTE(0, 0);                                                    \
    MC_STORE_A(1);                                                       \
    MC_ORDER_FIRST();                                                    \
    __syncthreads();                                                     \
    __builtin_amdgcn_sched_barrier(0);                                   \
    MC_LOAD_A(2 * s_next);                                               \
    MC_COMPUTE(1, 1);                                                    \
    MC_STORE_B();                                                        \
    MC_STORE_A(0);                                                       \
    b_st ^= 2 * kBStage;                                                 \
    b_rd ^= 2 * kBStage;                                                 \
    MC_ORDER_SECOND();                                                   \
    __syncthreads();                                                     \
    __builtin_amdgcn_sched_barrier(0);                                   \
  }

  acc16 acc[4][2];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][mb][r] = 0.f;

  {
    if (ragged && s_begin + 1 == rounds) MC_DROP_MISSING_CHANNELS();
    MC_LOAD_B(s_begin);
    MC_LOAD_A(2 * s_begin);
    MC_STORE_A(0);
    b_st ^= 2 * kBStage;  // (MC_STORE_B fills the buffer the products do not read)
    MC_STORE_B();
    b_st ^= 2 * kBStage;
    __syncthreads();
    for (int s = s_begin; s < s_end; ++s) {
      if (ragged && s + 2 == rounds) MC_DROP_MISSING_CHANNELS();
      MC_ROUND(s);
    }
  }
#undef MC_LOADF
#undef MC_LOAD_A
#undef MC_LOAD_B
#undef MC_DROP_MISSING_CHANNELS
#undef MC_STORE_A
#undef MC_STORE_B
#undef MC_COMPUTE
#undef MC_ORDER_FIRST
#undef MC_ORDER_SECOND
#undef MC_SG
#undef MC_ROUND

  // Finish.  Y = A^T m A, A^T = [1 1 1 0; 0 1 -1 -1].  This wavefront holds row i =
  // wave of m (columns j = 0 .. 3): the sums over j stay in registers,
  //   s[0] = m0 + m1 + m2,  s[1] = m1 - m2 - m3,
  // and go to Es[dj][i][co][t]; accumulator register r of lane l is channel
  // 32 mb + 8 (r / 4) + 4 (l / 32) + r % 4, block l % 32.
  float sv[2][2][16];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float m0 = acc[0][mb][r], m1 = acc[1][mb][r], m2 = acc[2][mb][r], m3 = acc[3][mb][r];
      sv[0][mb][r] = m0 + m1 + m2;
      sv[1][mb][r] = m1 - m2 - m3;
    }
  __syncthreads();  // every wavefront is done with the stage buffers
  if (a.counters != nullptr) {
    // The partial sums and the counter are accessed with device-scope atomic operations
    // only (relaxed stores and loads that go past the per-XCD L2, which is not coherent
    // with the other seven), so no cache write-back or invalidation is needed: a
    // workgroup waits until its own stores have completed and then counts.  (A
    // device-scope store is written through to the memory side and counted down by vmcnt
    // when acknowledged there; the relaxed accesses alone promise nothing of the kind.)
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx942__) && !defined(__gfx950__)
#error "the in-launch sum of channel slices relies on gfx942 / gfx950 device-scope write-through"
#endif
    const int tile_id = blockIdx.x;
    const size_t slice_elems = static_cast<size_t>(gridDim.x) * (64 * 256);
    float* mine = a.partial + blockIdx.y * slice_elems + static_cast<size_t>(tile_id) * (64 * 256) + tid;
#pragma unroll
    for (int v = 0; v < 64; ++v)
      __hip_atomic_store(mine + v * 256, sv[v >> 5][(v >> 4) & 1][v & 15], __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's partial sums have arrived
    __syncthreads();                                   // ... and every thread's
    int* arrived = reinterpret_cast<int*>(lds);
    if (tid == 0)
      arrived[0] = __hip_atomic_fetch_add(&a.counters[tile_id], 1, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const int before = arrived[0];
    __syncthreads();  // (lds is about to be reused)
    if (before != static_cast<int>(gridDim.y) - 1) return;  // uniform over the workgroup
    // the next launch on this stream starts from zero
    if (tid == 0)
      __hip_atomic_store(&a.counters[tile_id], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float* part = a.partial + static_cast<size_t>(tile_id) * (64 * 256) + tid;
#pragma unroll
    for (int v = 0; v < 64; ++v)
      sv[v >> 5][(v >> 4) & 1][v & 15] =
          __hip_atomic_load(part + v * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (unsigned z = 1; z < gridDim.y; ++z) {
      part += slice_elems;
#pragma unroll
      for (int v = 0; v < 64; ++v)
        sv[v >> 5][(v >> 4) & 1][v & 15] +=
            __hip_atomic_load(part + v * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  float* const Es = lds;
#pragma unroll
  for (int dj = 0; dj < 2; ++dj)
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int co = 32 * mb + 8 * (r / 4) + 4 * lhi + (r % 4);
        Es[((dj * 4 + wave) * kTileM + co) * kTileT + l32] = sv[dj][mb][r];
      }
  __syncthreads();

  // Thread = (block tid % 32, channels tid / 32 + 8 q): the sums over the four rows,
  //   out[0][dj] = s0 + s1 + s2,  out[1][dj] = s1 - s2 - s3,
  // then the layer's epilogue on the up to four outputs of the block inside the map.
  const int tq = tid & 31, cq = tid >> 5;
  const int t = nt * kTileT + tq;
  if (t >= a.T) return;
  const int n = fast_div(t, a.div_img_mul, a.div_img_shift);
  const int rem = t - n * a.ThTw;
  const int ty = fast_div(rem, a.div_tw_mul, a.div_tw_shift);
  const int tx = rem - ty * a.Tw;
  const int ho = 2 * ty, wo = 2 * tx;
  const bool row1 = ho + 1 < a.Ho, col1 = wo + 1 < a.Wo;
  const int c_second = a.Cout - a.c_first;
#pragma unroll 2
  for (int q = 0; q < 8; ++q) {
    const int cl = cq + 8 * q;
    const int c = mt * kTileM + cl;
    if (c >= a.Cout) break;
    float out[2][2];
#pragma unroll
    for (int dj = 0; dj < 2; ++dj) {
      const float s0 = Es[((dj * 4 + 0) * kTileM + cl) * kTileT + tq];
      const float s1 = Es[((dj * 4 + 1) * kTileM + cl) * kTileT + tq];
      const float s2 = Es[((dj * 4 + 2) * kTileM + cl) * kTileT + tq];
      const float s3 = Es[((dj * 4 + 3) * kTileM + cl) * kTileT + tq];
      out[0][dj] = s0 + s1 + s2;
      out[1][dj] = s1 - s2 - s3;
    }
    const float sc = a.scale ? a.scale[c] : 1.f;
    const float sh = a.shift ? a.shift[c] : 0.f;
    const bool first = c < a.c_first;
    float* __restrict__ yc = first ? a.y : a.y_second;
    const long base = first ? (((long)n * a.c_first + c) * a.Ho + ho) * a.Wo + wo
                            : (((long)n * c_second + (c - a.c_first)) * a.Ho + ho) * a.Wo + wo;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      out[i][0] = out[i][0] * sc + sh;
      out[i][1] = out[i][1] * sc + sh;
    }
    if (a.pairs) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (i == 1 && !row1) break;
        const long o = base + i * a.Wo;
        float2 val = make_float2(out[i][0], out[i][1]);
        if (a.residual) {
          const float2 r = *reinterpret_cast<const float2*>(a.residual + o);
          val.x += r.x;
          val.y += r.y;
        }
        val.x = act_value(val.x, a.act, a.slope);
        val.y = act_value(val.y, a.act, a.slope);
        *reinterpret_cast<float2*>(yc + o) = val;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (i == 1 && !row1) break;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (j == 1 && !col1) break;
          const long o = base + i * a.Wo + j;
          float val = out[i][j];
          if (a.residual) val += a.residual[o];
          yc[o] = act_value(val, a.act, a.slope);
        }
      }
    }
  }
}

}  // namespace

struct WinogradState {
  mcConvGeom geom;
  int Ho = 0, Wo = 0;
  int MT = 0, KT = 0;
  float* u = nullptr;  // packed transformed filters, allocated when weights first arrive
  bool have_weights = false;
};

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
  w->MT = ceil_div(g.channels_out, kTileM);
  w->KT = 2 * ceil_div(g.channels_in, 2 * kStageC);
  return w;
}

void winograd_destroy(WinogradState* w) {
  if (!w) return;
  if (w->u) (void)hipFree(w->u);
  delete w;
}

// Whether one image can take this path at all: bottom, top and the packed filters
// are addressed with 31-bit byte offsets.
bool winograd_fits(const WinogradState* w, int /*num*/) {
  const mcConvGeom& g = w->geom;
  const long in_img = (long)g.channels_in * g.height_in * g.width_in;
  const long out_img = (long)g.channels_out * w->Ho * w->Wo;
  const long u_floats = (long)w->MT * w->KT * kAStage;
  return in_img < (1L << 29) && out_img < (1L << 29) && u_floats < (1L << 29);
}

// The automatic choice.  Per output block the direct path multiplies 36 Cin Cout
// times, this path 16 Cin Cout times; both read the bottom and write the top once.
// Measured, this path against the direct one: launches of some size win whenever both
// channel counts reach 64 (64 -> 64 on 56x56, batch 64: 97 us against 128; 128 -> 128
// on 28x28: 95 / 141; 256 -> 256 on 14x14: 91 / 148; 512 -> 512 on 7x7, which pads to
// 8x8: 101 / 156; VGG's 64 -> 64 on 300x300, batch 8: 295 / 423, 512 -> 512 on 38x38:
// 245 / 430; the RPN head 1024 -> 512 on 38x63: 110 / 197; SSD's merged heads 512 -> 100
// on 38x38: 86 / 124, 1024 -> 150 on 19x19: 66 / 97, 512 -> 150 on 10x10: 35 / 39).
// What loses: 32 input channels (the loop is four rounds long: 56 / 47 us), an
// output tile that is half padding (64 -> 32: 86 / 82), and launches of a few tiles,
// whose time is this kernel's longer prologue and finish (256 -> 150 on 5x5 maps, 9
// tiles: 25 / 19 us; one image of 256 channels on 14x14: 22 / 19; config 1's single
// 64 -> 64 layer on one 56x56 image, 25 tiles of 8 rounds: 17 / 12).
bool winograd_pays(const WinogradState* w, int num) {
  const mcConvGeom& g = w->geom;
  const long blocks = (long)num * ((w->Ho + 1) / 2) * ((w->Wo + 1) / 2);
  if (g.channels_in < 64) return false;
  if (4 * g.channels_out < 3 * w->MT * kTileM) return false;
  // odd and tiny maps compute blocks that hang over the edge: a 3x3 map is four
  // blocks for nine outputs (16 x 4 products against 36 x 9 / 4 useful ones)
  if (10L * w->Ho * w->Wo < 26L * ((w->Ho + 1) / 2) * ((w->Wo + 1) / 2)) return false;
  const long tiles = (long)w->MT * ceil_div(blocks, kTileT);
  return tiles * (w->KT / 2) >= 1200;
}

int winograd_set_weights(WinogradState* w, const float* weights, hipStream_t st) {
  const long floats = (long)w->MT * w->KT * kAStage;
  if (!w->u) MC_HIP(hipMalloc(&w->u, sizeof(float) * floats));
  const long threads = (long)w->MT * kTileM * w->KT * kStageC;
  winograd_pack_filter_kernel<<<static_cast<unsigned>(ceil_div(threads, 256)), 256, 0, st>>>(
      weights, w->u, w->geom.channels_out, w->geom.channels_in, w->MT, w->KT);
  MC_LAUNCH_CHECK();
  w->have_weights = true;
  return 0;
}

double winograd_issued_flops(const WinogradState* w, int num) {
  const double blocks = (double)num * ((w->Ho + 1) / 2) * ((w->Wo + 1) / 2);
  return 2. * 16. * w->geom.channels_in * w->geom.channels_out * blocks;
}

int winograd_forward(WinogradState* w, int num, const float* bottom, float* top,
                     const mcEpilogue* ep, void* stream, float* top_second, int c_first,
                     int images_per_run, int forced_slices) {
  MC_REQUIRE(w->have_weights, "mcConvForward: the plan has no weights yet");
  MC_REQUIRE(!top_second || (c_first > 0 && c_first < w->geom.channels_out && !(ep && ep->residual)),
             "mcConvForwardTwoTops: needs group 1, a split inside the output channels and no "
             "residual");
  if (!top_second) c_first = w->geom.channels_out;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const mcConvGeom& g = w->geom;
  const long in_img = (long)g.channels_in * g.height_in * g.width_in;
  const long hw_out = (long)w->Ho * w->Wo;
  const long top_img = (long)g.channels_out * hw_out;
  const long out_img = c_first * hw_out, second_img = (g.channels_out - c_first) * hw_out;
  const int Th = (w->Ho + 1) / 2, Tw = (w->Wo + 1) / 2;
  // equal runs of whole images that the 31-bit byte offsets reach
  const long lim = (1L << 29) - 1;
  long per = std::min(lim / in_img, lim / top_img);
  per = std::min(per, lim / ((long)Th * Tw));
  if (images_per_run > 0) per = std::min<long>(per, images_per_run);
  MC_REQUIRE(per >= 1, "mcConvForward: a single image exceeds 2^29 elements");
  const int runs = ceil_div(num, per);
  const int run_len = ceil_div(num, runs);

  WinogradArgs a;
  a.u = w->u;
  a.u_bytes = static_cast<unsigned>(sizeof(float) * (long)w->MT * w->KT * kAStage);
  a.scale = ep ? ep->scale : nullptr;
  a.shift = ep ? ep->shift : nullptr;
  a.C = g.channels_in;
  a.H = g.height_in;
  a.W = g.width_in;
  a.HW = g.height_in * g.width_in;
  a.x_nstride = static_cast<int>(in_img);
  a.Cout = g.channels_out;
  a.Ho = w->Ho;
  a.Wo = w->Wo;
  a.HoWo = static_cast<int>(hw_out);
  a.pad_h = g.pad_h;
  a.pad_w = g.pad_w;
  a.Tw = Tw;
  a.ThTw = Th * Tw;
  a.MT = w->MT;
  a.KT = w->KT;
  a.c_first = c_first;
  a.act = ep ? ep->activation : MC_ACT_NONE;
  a.slope = ep ? ep->negative_slope : 0.f;
  // (top and residual rows are 8-byte aligned when the width is even and the blob is)
  a.pairs = w->Wo % 2 == 0 && reinterpret_cast<uintptr_t>(top) % 8 == 0 &&
            reinterpret_cast<uintptr_t>(top_second) % 8 == 0 &&
            (!ep || !ep->residual || reinterpret_cast<uintptr_t>(ep->residual) % 8 == 0);
  for (int n0 = 0; n0 < num; n0 += run_len) {
    const int n = std::min(run_len, num - n0);
    a.x = bottom + n0 * in_img;
    a.x_bytes = static_cast<unsigned>(n * in_img * 4);
    a.y = top + n0 * out_img;
    a.y_second = top_second ? top_second + n0 * second_img : nullptr;
    a.residual = (ep && ep->residual) ? ep->residual + n0 * out_img : nullptr;
    a.T = n * a.ThTw;
    a.NT = ceil_div(a.T, kTileT);
    make_fast_div(a.ThTw, (unsigned long long)a.NT * kTileT + 1, &a.div_img_mul, &a.div_img_shift);
    make_fast_div(a.Tw, (unsigned long long)a.ThTw + 1, &a.div_tw_mul, &a.div_tw_shift);
    make_fast_div(a.MT, (unsigned long long)a.MT * a.NT + 1, &a.div_mt_mul, &a.div_mt_shift);
    const long tiles = (long)a.MT * a.NT;
    MC_REQUIRE(tiles < (1L << 31), "mcConvForward: grid too large");
    // A launch that leaves workgroup slots empty (two per CU) cuts the channel rounds
    // into slices, each at least four rounds long.
    const int rounds = w->KT / 2;
    int slices = forced_slices > 0 ? forced_slices : static_cast<int>(2L * kNumCu / tiles);
    slices = std::max(1, std::min(std::min(slices, 16), forced_slices > 0 ? rounds : rounds / 4));
    a.rounds_per_slice = ceil_div(rounds, slices);
    slices = ceil_div(rounds, a.rounds_per_slice);  // no empty slice
    a.partial = nullptr;
    a.counters = nullptr;
    if (slices > 1) {
      if (stream_workspace(st, sizeof(float) * tiles * slices * 64 * 256, &a.partial)) return -1;
      if (stream_counters(st, static_cast<size_t>(tiles), &a.counters)) return -1;
    }
    const dim3 grid(static_cast<unsigned>(tiles), slices);
    winograd_fused_kernel<<<grid, 256, 0, st>>>(a);
    MC_LAUNCH_CHECK();
  }
  return 0;
}

}  // namespace mchip
