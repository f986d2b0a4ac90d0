// Implicit-GEMM Convolution / Deconvolution for gfx950 (fp32 MFMA).
//
// The contraction the reference performs per image as im2col + sgemm
// (reference src/layers/base_conv_layer.cpp:254-271, src/util/im2col.cpp:19-55)
// and, for Deconvolution, as sgemm(A^T) + col2im (base_conv_layer.cpp:280-296,
// im2col.cpp:153-187) is done here for the whole batch in one launch with no
// column buffer:
//
//   Y[g][m][p] = sum_k Wt[g][k][m] * X(p, k)      m = output channel in group
//                                                 p = (image, qh, qw) "pixel"
//                                                 k = (input channel, tap)
//
// X(p, k) is gathered straight from the NCHW bottom blob through a per-k tap
// table {element offset, dh, dw}; zero padding is a bounds test.  A
// Deconvolution with stride s is split into s_h*s_w output-parity classes, each
// of which is a stride-1 gather with its own tap table, so no scatter-add and
// no wasted multiply by inserted zeros.
//
// Tiling: 256 threads = 4 wavefronts per workgroup, BM x BN output tile,
// K step 16, LDS double buffer filled from registers (global loads for tile
// t+1 are in flight while tile t is multiplied).  Each wavefront owns a grid of
// 32x32 accumulators fed by v_mfma_f32_32x32x2_f32.  Filters are repacked once
// into K-major, zero-padded [g][Kpad][Mpad] so that A-tile loads are aligned
// float4 rows and need no predicates.
#include "conv_internal.h"
#include "mc_common.h"
#include "mchip/kernels.h"

#include <algorithm>
#include <cstring>
#include <vector>

namespace mchip {
namespace {

constexpr int BK = 16;
constexpr int LDK = BK + 4;  // LDS row pitch in floats

typedef float acc16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr int kModeMasks = 0, kModeOneMask = 1, kModePointwise = 2, kModePointwiseQuad = 3;
// Buffer descriptor word 3 for raw dword access on gfx9-family CDNA parts
// (32-bit data format, no swizzle, offsets checked against num_records).
constexpr int kBufferFlags = 0x00020000;
// VGPR offset that is out of range for every buffer this file builds (all are
// below 2 GiB) and still has room for the widest access without wrapping.
constexpr unsigned kNoElement = 0x80000000u;

struct IgemmArgs {
  const float* __restrict__ x;
  const float* __restrict__ wt;
  float* __restrict__ y;
  const int4* __restrict__ ktab;  // [Kpad] {byte offset, row-tap index, column-tap index, 0}
  const int* __restrict__ tap_dh;  // bottom row offset of row-tap index b
  const int* __restrict__ tap_dw;  // bottom column offset of column-tap index b
  int n_dh, n_dw;
  unsigned x_bytes, wt_bytes;      // extents for the buffer descriptors
  int pix_shift;                   // bytes added to pixel origins (x points that far before the blob)
  const float* __restrict__ scale;
  const float* __restrict__ shift;
  const float* __restrict__ residual;
  int P;              // pixels = num * Hq * Wq
  int Hq, Wq, HqWq;   // iteration grid of this sub-problem
  unsigned div_hw_mul, div_hw_shift;  // p / HqWq  as multiply-high and shift (shift 32: divisor 1)
  unsigned div_w_mul, div_w_shift;    // rem / Wq
  unsigned div_mt_mul, div_mt_shift;  // logical tile / MT
  unsigned y_bytes, c_bytes;          // top blob and per-channel vector extents (descriptors)
  int H, W;           // bottom height / width
  int q_sh, q_sw;     // bottom origin of pixel (qh,qw): qh*q_sh + in_oh
  int in_oh, in_ow;
  int K;              // rows of the gather before padding to a multiple of BK
  int x_cstride;      // H*W
  int x_nstride;      // Cin*H*W
  int x_gstride;      // (Cin/g)*H*W
  int M;              // output channels per group
  int Mpad, Kpad;
  int Wo;             // top width
  int y_cstride;      // Ho*Wo
  int y_nstride;      // Cout*Ho*Wo
  int out_sh, out_sw, out_oh, out_ow;  // top row = qh*out_sh + out_oh
  int MT, NT;         // tile counts
  int kt_per_split;   // K tiles per blockIdx.z slice (split-K)
  int split_stride;   // elements between the partial outputs of two slices
  // Slices summed inside the launch (counters != nullptr): every workgroup leaves
  // its accumulators in `partial` ([slice][tile][register][thread])
  // and counts in counters[tile]; the last one to arrive adds the slices in slice
  // order, runs the epilogue and puts the counter back to zero.
  float* partial;
  int* counters;
  int partial_tiles;  // tiles per slice in `partial`
  int act;
  float slope;
};

// Up to four sub-problems (the output-parity classes of a Deconvolution) run
// in one launch: blockIdx.z = sub-problem * slices + K slice.
constexpr int kMaxSubs = 4;
struct IgemmBatch {
  IgemmArgs sub[kMaxSubs];
  int slices;
};

__device__ __forceinline__ float f4at(const float4& v, int e) {
  return e == 0 ? v.x : (e == 1 ? v.y : (e == 2 ? v.z : v.w));
}

__device__ __forceinline__ float apply_act(float v, int act, float slope) {
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

// OCC = wavefronts per SIMD the register allocation must leave room for.
// MODE selects how the K loop finds and guards the elements it gathers:
//   kModeMasks     tap table + one "outside the image" bit mask per tap row and
//                  per tap column (any kernel up to 31 x 31 taps);
//   kModeOneMask   tap table + one mask with a bit per (row, column) tap pair,
//                  for kernels with at most 31 taps (3x3, 5x5) and a channel
//                  count that is a multiple of 4: the K rows are then ordered
//                  (channel block of 4, tap, channel in block), so the four
//                  rows a thread gathers per step share one tap and one
//                  validity test;
//   kModePointwise no table and no mask, see below;
//   kModePointwiseQuad  the same for stride 1 on planes of a multiple of four pixels with
//                  K a multiple of 16 (64-pixel tile only): a thread fetches four
//                  consecutive pixels of one channel with one 16-byte load instead of
//                  one pixel of four channels with four loads, and transposes them on
//                  the way into LDS (four 4-byte stores).  Same products, same order.
// Pointwise: every row k of the gather is channel k of the bottom blob
// at the thread's own pixel (1x1 kernel, no padding), so the K loop needs no
// tap table and no bounds handling at all.
// ONE_SUB: the launch holds one sub-problem (every Convolution): its arguments then sit
// at fixed places of the argument block and are fetched in one batch at the top, instead
// of after the number of slices has arrived and said which sub-problem this workgroup
// belongs to.
template <int BM, int BN, int WM, int WN, int OCC, int MODE, int KS, bool ONE_SUB = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void igemm_kernel(
    const IgemmBatch batch) {
  static_assert(WM * WN == 4, "four wavefronts per workgroup");
  int sub_index = 0, kslice = blockIdx.z;
  if constexpr (!ONE_SUB) {
    while (kslice >= batch.slices) {  // at most kMaxSubs - 1 rounds, on the scalar unit
      kslice -= batch.slices;
      ++sub_index;
    }
  }
  const IgemmArgs& a = batch.sub[sub_index];
  // sub-problems of one launch may differ in tile count: the grid is the largest
  // (a single sub-problem's grid is exact: no test, and no branch that keeps the argument
  // fetches behind it from being issued together)
  if constexpr (!ONE_SUB) {
    if (static_cast<int>(blockIdx.x) >= a.MT * a.NT) return;
  }
  static_assert(BN >= 64 && 256 % BN == 0, "BN must be 64, 128 or 256");
  constexpr int TM = BM / WM / 32;
  constexpr int TN = BN / WN / 32;
  static_assert(TM >= 1 && TN >= 1, "wave tile must hold a 32x32 block");
  constexpr int QUADS = BK / 4;                   // float4 groups along K per tile
  constexpr int ROWS_PER_PASS = 256 / BN;         // K quads gathered per pass
  constexpr int B_Q = QUADS / ROWS_PER_PASS;      // quads per thread
  static_assert(B_Q >= 1, "tile too narrow for 256 gathering threads");
  constexpr int A_F4 = BM * QUADS;                // float4 per A tile
  constexpr int A_VEC = (A_F4 + 255) / 256;

  // K runs fastest in LDS ([row][k], rows padded to LDK floats) so that one
  // ds_read_b128 hands a lane four K steps of its MFMA operand; the 80-byte row
  // pitch spreads eight consecutive rows over all 32 banks.
  // KS 16-row K tiles form one stage (one barrier per stage).
  __shared__ __attribute__((aligned(16))) float As[2][KS][BM][LDK];
  __shared__ __attribute__((aligned(16))) float Bs[2][KS][BN][LDK];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = blockIdx.y;

  // XCD-aware tile order: workgroup ids are dealt round-robin to the 8 XCDs, so
  // give each XCD a contiguous run of logical tiles (m fastest): the tiles that
  // share one pixel tile, and neighbouring pixel tiles, then hit the same L2.
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

  // On this hardware ordinary vector ALU instructions and MFMA instructions of
  // co-resident wavefronts do not overlap: every VALU cycle in the K loop is
  // taken from the matrix pipe.  The loop therefore does its addressing on the
  // scalar unit and in the memory instructions themselves:
  //  * bottom and filter are read through buffer descriptors: scalar base,
  //    scalar offset per K row / K tile, one fixed VGPR offset per thread, and
  //    an out-of-range VGPR offset returns 0 without a branch or a select.
  //    Both buffers are kept below 2 GiB and "no element" is offset bit 31.  The
  //    bottom descriptor starts far enough before the blob that the sum of a
  //    pixel origin and a tap offset is never negative, so a flagged offset lies
  //    in [2^31, 2^32 - 16) and offset + access size cannot wrap around 2^32
  //    (an access that carries into bit 32 would leave the checked range);
  //  * per thread, bit b of row_bad / col_bad says that row (column) tap b
  //    falls outside the image for this thread's pixel, so an element costs two
  //    bit-field extracts, an add and two shift-ors (nothing at all when PW);
  //  * the loop is unrolled over the two LDS buffers so every LDS address is
  //    a base register plus an immediate.
  const __amdgpu_buffer_rsrc_t xres =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.x), 0, a.x_bytes, kBufferFlags);
  const __amdgpu_buffer_rsrc_t wres =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.wt), 0, a.wt_bytes, kBufferFlags);

  // The pixel this thread gathers for the B tile (fixed over the K loop).
  const int pj = tid % BN;
  const int prow = tid / BN;  // wave-uniform because BN >= 64
  // byte offset of the pixel's origin from the descriptor base (never negative)
  constexpr bool PW4 = MODE == kModePointwiseQuad;  // pointwise, stride 1: four pixels of a channel per load
  constexpr bool PW = MODE == kModePointwise || PW4;
  static_assert(!PW4 || (BN == 64 && KS == 1), "the pixel-quad gather is built for the 64-pixel tile");
  unsigned xvoff = PW ? kNoElement : 0u;
  unsigned row_bad = 0xFFFFFFFFu, col_bad = 0xFFFFFFFFu;
  {
    // PW4: thread = (K row tid % 16, pixel quad tid / 16); the plane is a multiple of four
    // pixels, so a quad never straddles two images
    const int p = PW4 ? nt * BN + 4 * (tid >> 4) : nt * BN + pj;
    // (the divisions are prepared for every column of the last tile, also those past the
    // last pixel: the pointwise modes compute first and pick afterwards, without a branch)
    const int n = fast_div(p, a.div_hw_mul, a.div_hw_shift);
    const int rem = p - n * a.HqWq;
    // (the pixel-quad mode runs only where pixel `rem` of the iteration grid is element
    // `rem` of the bottom plane and of the top plane: no row and column needed)
    const int qh = PW4 ? 0 : fast_div(rem, a.div_w_mul, a.div_w_shift);
    const int qw = PW4 ? 0 : rem - qh * a.Wq;
    const int hi0 = qh * a.q_sh + a.in_oh;
    const int wi0 = qw * a.q_sw + a.in_ow;
    unsigned origin = static_cast<unsigned>(
        ((n * a.x_nstride + g * a.x_gstride + (PW4 ? rem : hi0 * a.W + wi0)) << 2) + a.pix_shift);
    if constexpr (PW4) origin += static_cast<unsigned>(tid & 15) * (static_cast<unsigned>(a.x_cstride) * 4u);
    if constexpr (PW) xvoff = p < a.P ? origin : kNoElement;
    if (!PW && p < a.P) {
      xvoff = origin;
      if constexpr (!PW) {
        row_bad = 0x80000000u;  // bit 31: the tap of K padding rows, never valid
        col_bad = 0u;
        for (int b = 0; b < a.n_dh; ++b)
          row_bad |= static_cast<unsigned>(static_cast<unsigned>(hi0 + a.tap_dh[b]) >=
                                           static_cast<unsigned>(a.H))
                     << b;
        for (int b = 0; b < a.n_dw; ++b)
          col_bad |= static_cast<unsigned>(static_cast<unsigned>(wi0 + a.tap_dw[b]) >=
                                           static_cast<unsigned>(a.W))
                     << b;
        if constexpr (MODE == kModeOneMask) {
          // bit i*n_dw + j = row tap i or column tap j outside; the result replaces row_bad
          const unsigned all_cols = (1u << a.n_dw) - 1u;
          unsigned pair_bad = 0x80000000u;
          for (int b = 0; b < a.n_dh; ++b)
            pair_bad |= (((row_bad >> b) & 1u) ? all_cols : col_bad) << (b * a.n_dw);
          row_bad = pair_bad;
        }
      }
    }
  }
  const int KT = a.Kpad / (BK * KS);  // stages
  // Split-K: slice z multiplies K stages [kt_begin, kt_end); its partial sums go
  // to the workspace the last workgroup of the tile adds up (IgemmArgs::partial)
  // or, for a launch with two tops, into its own copy of the top blob.
  const int kt_begin = kslice * a.kt_per_split;
  const int kt_end = min(KT, kt_begin + a.kt_per_split);
  float* __restrict__ yout = a.y + (size_t)kslice * a.split_stride;

  // Packed filter: [g][K tile][m][16 k], so an A tile is one contiguous run:
  // per-thread byte offset inside the tile, scalar byte offset of the tile.
  unsigned avoff[A_VEC];
#pragma unroll
  for (int i = 0; i < A_VEC; ++i) {
    const int f = tid + 256 * i;
    avoff[i] = (A_F4 % 256 == 0 || f < A_F4) ? static_cast<unsigned>((mt * BM * BK + f * 4) * 4)
                                              : kNoElement;
  }
  const unsigned wt_kt_bytes = static_cast<unsigned>(a.Mpad) * BK * 4;
  const unsigned wt_g_bytes = static_cast<unsigned>(g) * (a.Kpad / BK) * wt_kt_bytes;
  // (said to be uniform: the compiler otherwise merges this load with the one inside the
  // divergent branch above into a vector register, and every pixel-quad load of the K
  // loop, whose scalar offset is a multiple of it, gets wrapped in a loop over lanes)
  const unsigned x_cbytes = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(a.x_cstride) * 4);
  const int kmax = a.K - 1;

  float4 areg[KS][A_VEC];
  float4 breg[KS][B_Q];

#define MC_LOADF(res, voff, soff) \
  __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(res, voff, soff, 0))
#define MC_GATHER1(dst, t)                                                                   \
  {                                                                                          \
    /* The tap's byte offset rides in the scalar offset of the load; the VGPR                \
       offset is the pixel origin, with bit 31 set when the tap is outside the               \
       image.  Origin + tap offset stays below 2^31, so a flagged sum cannot wrap            \
       whether or not the hardware adds the scalar offset before its range check. */        \
    const unsigned rb = __builtin_amdgcn_ubfe(row_bad, (t).y, 1);                            \
    const unsigned cb = __builtin_amdgcn_ubfe(col_bad, (t).z, 1);                            \
    dst = MC_LOADF(xres, (cb << 31) | ((rb << 31) | xvoff), (t).x);                          \
  }
#define MC_LOAD_TILES(kt)                                                                    \
  _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                        \
    const int kt16 = (kt)*KS + ks;                                                           \
    const unsigned a_soff = wt_g_bytes + static_cast<unsigned>(kt16) * wt_kt_bytes;          \
    _Pragma("unroll") for (int i = 0; i < A_VEC; ++i) {                                      \
      const u32x4 w4 = __builtin_amdgcn_raw_buffer_load_b128(wres, avoff[i], a_soff, 0);     \
      areg[ks][i] = __builtin_bit_cast(float4, w4);                                          \
    }                                                                                        \
    _Pragma("unroll") for (int i = 0; i < B_Q; ++i) {                                        \
      const int krow =                                                                       \
          __builtin_amdgcn_readfirstlane(kt16 * BK + (i * ROWS_PER_PASS + prow) * 4);        \
      if constexpr (PW4) {                                                                   \
        /* K is a multiple of 16 here: no padding rows */                                    \
        const u32x4 q4 = __builtin_amdgcn_raw_buffer_load_b128(                              \
            xres, xvoff, static_cast<unsigned>(kt16 * BK) * x_cbytes, 0);                    \
        breg[ks][i] = __builtin_bit_cast(float4, q4);                                        \
      } else if constexpr (PW) {                                                             \
        /* padding rows re-read the last channel; their filter rows are zero */              \
        breg[ks][i].x = MC_LOADF(xres, xvoff, static_cast<unsigned>(min(krow, kmax)) * x_cbytes);\
        breg[ks][i].y =                                                                          \
            MC_LOADF(xres, xvoff, static_cast<unsigned>(min(krow + 1, kmax)) * x_cbytes);    \
        breg[ks][i].z =                                                                          \
            MC_LOADF(xres, xvoff, static_cast<unsigned>(min(krow + 2, kmax)) * x_cbytes);    \
        breg[ks][i].w =                                                                          \
            MC_LOADF(xres, xvoff, static_cast<unsigned>(min(krow + 3, kmax)) * x_cbytes);    \
      } else {                                                                               \
        const int4 t0 = a.ktab[krow], t1 = a.ktab[krow + 1], t2 = a.ktab[krow + 2],          \
                   t3 = a.ktab[krow + 3];                                                    \
        if constexpr (MODE == kModeOneMask) {                                                \
          /* rows krow .. krow+3: four channels at one tap */                                \
          const unsigned pb = __builtin_amdgcn_ubfe(row_bad, t0.w, 1);                       \
          const unsigned voff = (pb << 31) | xvoff;                                          \
          breg[ks][i].x = MC_LOADF(xres, voff, t0.x);                                            \
          breg[ks][i].y = MC_LOADF(xres, voff, t1.x);                                            \
          breg[ks][i].z = MC_LOADF(xres, voff, t2.x);                                            \
          breg[ks][i].w = MC_LOADF(xres, voff, t3.x);                                            \
        } else {                                                                             \
          MC_GATHER1(breg[ks][i].x, t0);                                                         \
          MC_GATHER1(breg[ks][i].y, t1);                                                         \
          MC_GATHER1(breg[ks][i].z, t2);                                                         \
          MC_GATHER1(breg[ks][i].w, t3);                                                         \
        }                                                                                    \
      }                                                                                      \
    }                                                                                        \
  }
#define MC_STORE_TILES(buf)                                                                  \
  _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                        \
    _Pragma("unroll") for (int i = 0; i < A_VEC; ++i) {                                      \
      const int f = tid + 256 * i;                                                           \
      if (A_F4 % 256 == 0 || f < A_F4)                                                       \
        *reinterpret_cast<float4*>(&As[buf][ks][f / QUADS][(f % QUADS) * 4]) = areg[ks][i];  \
    }                                                                                        \
    _Pragma("unroll") for (int i = 0; i < B_Q; ++i) {                                        \
      if constexpr (PW4) {                                                                   \
        float* col = &Bs[buf][ks][4 * (tid >> 4)][tid & 15];                                 \
        col[0] = breg[ks][i].x;                                                              \
        col[LDK] = breg[ks][i].y;                                                            \
        col[2 * LDK] = breg[ks][i].z;                                                        \
        col[3 * LDK] = breg[ks][i].w;                                                        \
      } else {                                                                               \
        *reinterpret_cast<float4*>(&Bs[buf][ks][pj][(i * ROWS_PER_PASS + prow) * 4]) =       \
            breg[ks][i];                                                                     \
      }                                                                                      \
    }                                                                                        \
  }
  // One MFMA K step multiplies k-pairs; which two physical k rows form a pair
  // is free as long as A and B agree, so half-wave 0 takes k = 8h+e and
  // half-wave 1 takes k = 8h+4+e for step (h, e): four steps per b128 read.
#define MC_COMPUTE(buf)                                                                      \
  _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                        \
    float4 av[TM][2], bv[TN][2];                                                             \
    _Pragma("unroll") for (int h = 0; h < 2; ++h) {                                          \
      _Pragma("unroll") for (int i = 0; i < TM; ++i) av[i][h] = *reinterpret_cast<           \
          const float4*>(&As[buf][ks][wm0 + i * 32 + l32][h * 8 + lhi * 4]);                 \
      _Pragma("unroll") for (int j = 0; j < TN; ++j) bv[j][h] = *reinterpret_cast<           \
          const float4*>(&Bs[buf][ks][wn0 + j * 32 + l32][h * 8 + lhi * 4]);                 \
    }                                                                                        \
    _Pragma("unroll") for (int h = 0; h < 2; ++h) {                                          \
      _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                        \
        _Pragma("unroll") for (int i = 0; i < TM; ++i) {                                     \
          _Pragma("unroll") for (int j = 0; j < TN; ++j) {                                   \
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(f4at(av[i][h], e),              \
                                                             f4at(bv[j][h], e), acc[i][j],   \
                                                             0, 0, 0);                       \
          }                                                                                  \
        }                                                                                    \
      }                                                                                      \
    }                                                                                        \
  }

  // Order of a stage's instructions inside a wavefront: the global loads of the next
  // stage (as a group the scheduler keeps first, not behind a hard scheduling barrier:
  // their scalar address arithmetic may mix with what follows), the LDS reads, three quarters
  // of the stage's MFMAs, the LDS stores of the next stage (which wait for its global
  // loads), the last quarter.  The last MFMAs work on registers only, so the compiler
  // lets them sink below the barrier that follows, next to the loads and LDS reads of
  // the next stage: a wavefront that arrives at the barrier still has matrix work in
  // flight.  With stores and barrier after the whole MFMA block (ResNet-50 b64, direct
  // path) 5.01 ms per forward, stores after half of the block 4.86, after a quarter
  // 4.91, after three quarters 4.87 (4.64 -> 4.54 with the Winograd layers).
#define MC_INTERLEAVE()                                                   \
  __builtin_amdgcn_sched_group_barrier(0x020, 32, 0);                     \
  __builtin_amdgcn_sched_group_barrier(0x100, 2 * KS * (TM + TN), 0);     \
  __builtin_amdgcn_sched_group_barrier(0x008, 6 * KS * TM * TN, 0);       \
  __builtin_amdgcn_sched_group_barrier(0x200, 16, 0);                     \
  __builtin_amdgcn_sched_group_barrier(0x008, 2 * KS * TM * TN, 0)

  acc16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int wm0 = (wave % WM) * (BM / WM);
  const int wn0 = (wave / WM) * (BN / WN);
  const int l32 = lane & 31;
  const int lhi = lane >> 5;

  // Per-channel factors of the epilogue: thread t < BM fetches the scale of row t of this
  // tile, thread BM + t its shift, before the K loop, and leaves them in the padding of
  // the first A buffer (columns BK and BK + 1 of row t, which no tile store and no
  // operand read touches) together with the first tile: the first barrier of the K loop
  // publishes them, and after the last MFMA a wavefront reads the (scale, shift) pairs of
  // its rows from there without another barrier and without waiting for the other three.
  float ep_val = tid < BM ? 1.f : 0.f;
  // Both pointers as scalars first: picking between the two *fields* makes the compiler
  // pick between their addresses in the argument block and fetch the pointer with a
  // vector load, a memory round trip every wavefront then waits for before it has
  // requested its first tile.
  const float* scale_ptr = a.scale;
  const float* shift_ptr = a.shift;
  asm("" : "+s"(scale_ptr), "+s"(shift_ptr));
#define MC_LOAD_FACTORS()                                                              \
  {                                                                                    \
    const float* src = tid < BM ? scale_ptr : shift_ptr;                               \
    const int row = mt * BM + (tid < BM ? tid : tid - BM);                             \
    if (tid < 2 * BM && src != nullptr && row < a.M) ep_val = src[g * a.M + row];      \
  }

  MC_LOAD_FACTORS();
#undef MC_LOAD_FACTORS
  static_assert(2 * BM <= 256 && LDK >= BK + 2, "factors go to the padding of the first A buffer");
#define MC_STORE_FACTORS() \
  if (tid < 2 * BM) As[0][0][tid & (BM - 1)][BK + (tid >= BM ? 1 : 0)] = ep_val
  if (kt_end > kt_begin) {
    // Tile kt_begin + t sits in LDS buffer t % 2; the loads of the next tile
    // are in flight while the MFMA block of the current one runs.
    const int nk = kt_end - kt_begin;
    MC_LOAD_TILES(kt_begin);
    MC_STORE_TILES(0);
    MC_STORE_FACTORS();
    __syncthreads();
    int t = 0;
    for (; t + 2 < nk; t += 2) {
      MC_LOAD_TILES(kt_begin + t + 1);
      MC_COMPUTE(0);
      MC_STORE_TILES(1);
      MC_INTERLEAVE();
      __syncthreads();
      MC_LOAD_TILES(kt_begin + t + 2);
      MC_COMPUTE(1);
      MC_STORE_TILES(0);
      MC_INTERLEAVE();
      __syncthreads();
    }
    // one or two tiles left; tile t is in buffer 0
    if (t + 1 < nk) {
      MC_LOAD_TILES(kt_begin + t + 1);
      MC_COMPUTE(0);
      MC_STORE_TILES(1);
      MC_INTERLEAVE();
      __syncthreads();
      MC_COMPUTE(1);
    } else {
      MC_COMPUTE(0);
    }
  } else {
    // (a slice past the last K tile of a short sub-problem: zeros, but it may be the one
    // that sums the slices and runs the epilogue)
    MC_STORE_FACTORS();
    __syncthreads();
  }
#undef MC_STORE_FACTORS
#undef MC_LOADF
#undef MC_GATHER1
#undef MC_LOAD_TILES
#undef MC_STORE_TILES
#undef MC_COMPUTE
#undef MC_INTERLEAVE

  // What the epilogue reads from the argument block is fetched here in one batch:
  // fetched where it is first used, the fields cost the wavefront four or five
  // scalar-memory round trips after the last MFMA, one after the other.  (Before the K
  // loop they would not fit the scalar registers the loop needs.)
  struct {
    int* counters;
    const float* residual;
    unsigned y_bytes, div_hw_mul, div_hw_shift, div_w_mul, div_w_shift;
    int y_cstride, y_nstride, Wo, out_sh, out_sw, out_oh, out_ow, M, P, HqWq, Wq, act;
    float slope;
  } e = {a.counters, a.residual, a.y_bytes, a.div_hw_mul, a.div_hw_shift, a.div_w_mul, a.div_w_shift,
         a.y_cstride, a.y_nstride, a.Wo, a.out_sh, a.out_sw, a.out_oh, a.out_ow, a.M, a.P, a.HqWq, a.Wq,
         a.act, a.slope};
  asm volatile("" ::"s"(e.counters), "s"(e.residual), "s"(e.y_bytes), "s"(e.div_hw_mul), "s"(e.div_hw_shift),
               "s"(e.div_w_mul), "s"(e.div_w_shift), "s"(e.y_cstride), "s"(e.y_nstride), "s"(e.Wo),
               "s"(e.out_sh), "s"(e.out_sw), "s"(e.out_oh), "s"(e.out_ow), "s"(e.M), "s"(e.P), "s"(e.HqWq),
               "s"(e.Wq), "s"(e.act), "s"(e.slope));

  if (e.counters != nullptr) {
    // K slices summed here: see IgemmArgs::partial.  The partial sums and the
    // counter are accessed with device-scope atomic operations only (relaxed
    // stores and loads that go past the per-XCD L2, which is not coherent with
    // the other seven), so no cache write-back or invalidation is needed: a
    // workgroup waits until its own stores have completed and then counts.
    // What this rests on is particular to the parts it is built for: a store with
    // device scope (sc1) is written through to the memory side, where all XCDs meet,
    // and vmcnt counts it down only when that write has been acknowledged; an
    // atomic on the counter issued after the wait is therefore ordered behind the
    // partial sums at the one place every later device-scope load reads from.  The
    // language's memory model promises none of this for relaxed accesses.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx942__) && !defined(__gfx950__)
#error "the in-launch sum of K slices relies on gfx942 / gfx950 device-scope write-through"
#endif
    const int tile_id = (sub_index * gridDim.y + g) * gridDim.x + blockIdx.x;
    constexpr int kRegs = TM * TN * 16;  // accumulator registers per thread
    float* mine = a.partial +
                  (static_cast<size_t>(kslice) * a.partial_tiles + tile_id) * (kRegs * 256) + tid;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          __hip_atomic_store(mine + ((i * TN + j) * 16 + r) * 256, acc[i][j][r], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's partial sums have arrived
    __syncthreads();  // ... every thread's, and every wave is done with the tiles in LDS
    int* arrived = reinterpret_cast<int*>(&As[0][0][0][0]);
    if (tid == 0)
      arrived[0] = __hip_atomic_fetch_add(&e.counters[tile_id], 1, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrived[0] != batch.slices - 1) return;  // uniform over the workgroup
    // the next launch on this stream starts from zero
    if (tid == 0)
      __hip_atomic_store(&e.counters[tile_id], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float* part = a.partial + static_cast<size_t>(tile_id) * (kRegs * 256) + tid;
    const size_t slice_elems = static_cast<size_t>(a.partial_tiles) * (kRegs * 256);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[i][j][r] = __hip_atomic_load(part + ((i * TN + j) * 16 + r) * 256, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
    for (int z = 1; z < batch.slices; ++z) {
      part += slice_elems;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            acc[i][j][r] += __hip_atomic_load(part + ((i * TN + j) * 16 + r) * 256, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
    }
  }

  // Epilogue.  Accumulator register r of lane l holds row 8*(r/4)+4*(l/32)+r%4,
  // column l%32 of its 32x32 block; a half-wave therefore stores 32 consecutive
  // pixels of one output channel.  Like the K loop it addresses through buffer
  // descriptors: one VGPR offset per lane (bit 31 set for a column past the last
  // pixel, which drops its stores), the row as a scalar offset.  Per-channel
  // factors and residual values are fetched eight rows at a time, all loads of
  // a batch issued before the first use.
  const bool has_scale = scale_ptr != nullptr;
  const bool has_shift = shift_ptr != nullptr;
  const bool has_res = e.residual != nullptr;
  const __amdgpu_buffer_rsrc_t yres =
      __builtin_amdgcn_make_buffer_rsrc(yout, 0, e.y_bytes, kBufferFlags);
  const __amdgpu_buffer_rsrc_t rres = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(e.residual), 0, has_res ? e.y_bytes : 0, kBufferFlags);
  // 0: none, 1: ReLU (max with 0), 2: leaky ReLU, 3: TanH / Sigmoid
  const int act_mode = e.act == MC_ACT_NONE ? 0
                       : e.act == MC_ACT_RELU ? (e.slope == 0.f ? 1 : 2)
                                              : 3;
  const unsigned cs4 = static_cast<unsigned>(e.y_cstride) * 4;
#define MC_ROW(r) (8 * ((r) / 4) + ((r) % 4))
#define MC_LOADF(res, voff, soff) \
  __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(res, voff, soff, 0))
#define MC_STORE_ROWS(EXPR)                                                                  \
  _Pragma("unroll") for (int q = 0; q < 8; ++q) {                                            \
    const float v = acc[i][j][half * 8 + q];                                                 \
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, (EXPR)), yres, y_voff,\
                                          MC_ROW(half * 8 + q) * cs4, 0);                    \
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int p = nt * BN + wn0 + j * 32 + l32;
    const int n = fast_div(p, e.div_hw_mul, e.div_hw_shift);
    const int rem = p - n * e.HqWq;
    int ybase;
    if constexpr (PW4) {
      ybase = n * e.y_nstride + rem;
    } else {
      const int qh = fast_div(rem, e.div_w_mul, e.div_w_shift);
      const int qw = rem - qh * e.Wq;
      ybase = n * e.y_nstride + (qh * e.out_sh + e.out_oh) * e.Wo + qw * e.out_sw + e.out_ow;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int mblock = mt * BM + wm0 + i * 32;  // wave-uniform
      const int m0 = mblock + 4 * lhi;
      if (mblock + 32 <= e.M) {
        // All 32 rows are real channels.
        const unsigned c0 = g * e.M + m0;
        const unsigned y_voff =
            p < e.P ? static_cast<unsigned>(ybase + c0 * e.y_cstride) * 4 : kNoElement;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          if (has_scale | has_shift) {
            float sc[8], sh[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
              const int lrow = wm0 + i * 32 + 4 * lhi + MC_ROW(half * 8 + q);
              const float2 f = *reinterpret_cast<const float2*>(&As[0][0][lrow][BK]);
              sc[q] = f.x;
              sh[q] = f.y;
            }
#pragma unroll
            for (int q = 0; q < 8; ++q)
              acc[i][j][half * 8 + q] = acc[i][j][half * 8 + q] * sc[q] + sh[q];
          }
          if (has_res) {
            float rs[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) rs[q] = MC_LOADF(rres, y_voff, MC_ROW(half * 8 + q) * cs4);
#pragma unroll
            for (int q = 0; q < 8; ++q) acc[i][j][half * 8 + q] += rs[q];
          }
          if (act_mode == 0) {
            MC_STORE_ROWS(v)
          } else if (act_mode == 1) {
            MC_STORE_ROWS(fmaxf(v, 0.f))
          } else if (act_mode == 2) {
            MC_STORE_ROWS(v > 0.f ? v : v * e.slope)
          } else {
            MC_STORE_ROWS(apply_act(v, e.act, e.slope))
          }
        }
      } else if (p < e.P) {
        // Block straddles the last channel: row by row, skipping rows >= M.
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + MC_ROW(r);
          if (m < e.M) {
            const int c = g * e.M + m;
            float v = acc[i][j][r];
            if (has_scale) v *= a.scale[c];
            if (has_shift) v += a.shift[c];
            const int yo = ybase + c * e.y_cstride;
            if (has_res) v += e.residual[yo];
            yout[yo] = apply_act(v, e.act, e.slope);
          }
        }
      }
    }
  }
#undef MC_ROW
#undef MC_LOADF
#undef MC_STORE_ROWS
}

// Split-K tail for a launch whose output channels belong to two blobs (two
// sibling layers computed together): v = act((sum over slices, in slice order) *
// scale[c] + shift[c]); channels [0, c_first) of every image go to y_first
// [num, c_first, plane], the others to y_second.  One thread per element; such
// outputs are small (detection heads).
__global__ __launch_bounds__(256) void splitk_reduce_two_kernel(
    const float* __restrict__ part, int slices, long slice_stride, long count,
    float* __restrict__ y_first, float* __restrict__ y_second, int c_first,
    const float* __restrict__ scale, const float* __restrict__ shift, int plane, int C, int act,
    float slope) {
  const long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x;
  if (i >= count) return;
  float v = part[i];
  for (int z = 1; z < slices; ++z) v += part[z * slice_stride + i];
  const unsigned iu = static_cast<unsigned>(i);  // count < 2^29
  const unsigned row = iu / static_cast<unsigned>(plane);  // n * C + c
  const unsigned p = iu - row * plane;
  const unsigned n = row / static_cast<unsigned>(C);
  const int c = static_cast<int>(row - n * C);
  if (scale) v *= scale[c];
  if (shift) v += shift[c];
  v = apply_act(v, act, slope);
  if (c < c_first)
    y_first[(static_cast<long>(n) * c_first + c) * plane + p] = v;
  else
    y_second[(static_cast<long>(n) * (C - c_first) + (c - c_first)) * plane + p] = v;
}

// Convolutions with at most kThinM output channels per group (the image-producing
// last layer of a generator, a one-channel score map): a 32-row MFMA tile would
// multiply mostly padding, and the layer is bound by reading its bottom blob
// anyway.  One thread per output pixel walks the K rows of the same gather
// (same tap table, same packed filter, read through scalar loads) and keeps the
// kThinM sums in registers; neighbouring threads read neighbouring addresses.
constexpr int kThinM = 4;
constexpr int kThinPx = 2;  // output pixels per thread: the scalar loads of a K row serve both
__global__ __launch_bounds__(256) void thin_conv_kernel(const IgemmBatch batch, int pointwise) {
  const IgemmArgs& a = batch.sub[blockIdx.z];
  const int g = blockIdx.y;
  // the gather of igemm_kernel's kModeMasks: pixel origin in the VGPR offset of a
  // buffer load, tap offset in its scalar offset, bit 31 for "outside the image"
  const __amdgpu_buffer_rsrc_t xres =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.x), 0, a.x_bytes, kBufferFlags);
  // pixel j of this thread is gridDim.x * 256 pixels after pixel j - 1, so the
  // lanes of a wavefront stay on neighbouring pixels
  int pix[kThinPx];
  unsigned xvoff[kThinPx], row_bad[kThinPx], col_bad[kThinPx];
  long ybase[kThinPx];
#pragma unroll
  for (int j = 0; j < kThinPx; ++j) {
    const int p = (j * static_cast<int>(gridDim.x) + static_cast<int>(blockIdx.x)) * 256 + threadIdx.x;
    pix[j] = p;
    xvoff[j] = kNoElement;
    row_bad[j] = 0xFFFFFFFFu;
    col_bad[j] = 0xFFFFFFFFu;
    ybase[j] = 0;
    if (p < a.P) {
      const int n = fast_div(p, a.div_hw_mul, a.div_hw_shift);
      const int rem = p - n * a.HqWq;
      const int qh = fast_div(rem, a.div_w_mul, a.div_w_shift);
      const int qw = rem - qh * a.Wq;
      const int hi0 = qh * a.q_sh + a.in_oh;
      const int wi0 = qw * a.q_sw + a.in_ow;
      xvoff[j] = static_cast<unsigned>(
          ((n * a.x_nstride + g * a.x_gstride + hi0 * a.W + wi0) << 2) + a.pix_shift);
      unsigned rb = 0x80000000u, cb = 0u;
      for (int b = 0; b < a.n_dh; ++b)
        rb |= static_cast<unsigned>(static_cast<unsigned>(hi0 + a.tap_dh[b]) >= static_cast<unsigned>(a.H)) << b;
      for (int b = 0; b < a.n_dw; ++b)
        cb |= static_cast<unsigned>(static_cast<unsigned>(wi0 + a.tap_dw[b]) >= static_cast<unsigned>(a.W)) << b;
      row_bad[j] = rb;
      col_bad[j] = cb;
      ybase[j] = static_cast<long>(n) * a.y_nstride +
                 static_cast<long>(qh * a.out_sh + a.out_oh) * a.Wo + qw * a.out_sw + a.out_ow;
    }
  }
  const float* __restrict__ wg = a.wt + static_cast<size_t>(g) * a.Kpad * a.Mpad;
  float acc[kThinPx][kThinM];
#pragma unroll
  for (int j = 0; j < kThinPx; ++j)
#pragma unroll
    for (int m = 0; m < kThinM; ++m) acc[j][m] = 0.f;
#define MC_LOADF(res, voff, soff) \
  __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(res, voff, soff, 0))
  // K in tiles of 16 over the padded extent (padding rows have zero filters and,
  // with a tap table, the never-valid tap): per tile the 4 x 16 filter values and
  // the 16 table entries are contiguous, so they arrive in a few wide scalar loads.
  const int kmax = a.K - 1;
  const unsigned x_cbytes = static_cast<unsigned>(a.x_cstride) * 4;
  for (int k0 = 0; k0 < a.Kpad; k0 += BK) {
    const float* __restrict__ wk = wg + (k0 >> 4) * (a.Mpad * BK);
    float v[kThinPx][BK];
    if (pointwise) {
#pragma unroll
      for (int i = 0; i < BK; ++i) {
        const unsigned soff = static_cast<unsigned>(min(k0 + i, kmax)) * x_cbytes;
#pragma unroll
        for (int j = 0; j < kThinPx; ++j) v[j][i] = MC_LOADF(xres, xvoff[j], soff);
      }
    } else {
      const int4* __restrict__ tk = a.ktab + k0;
#pragma unroll
      for (int i = 0; i < BK; ++i) {
        const int4 t = tk[i];
#pragma unroll
        for (int j = 0; j < kThinPx; ++j) {
          const unsigned rb = __builtin_amdgcn_ubfe(row_bad[j], t.y, 1);
          const unsigned cb = __builtin_amdgcn_ubfe(col_bad[j], t.z, 1);
          v[j][i] = MC_LOADF(xres, (cb << 31) | ((rb << 31) | xvoff[j]), t.x);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < BK; ++i) {
#pragma unroll
      for (int m = 0; m < kThinM; ++m) {
        const float w = wk[m * BK + i];
#pragma unroll
        for (int j = 0; j < kThinPx; ++j) acc[j][m] += w * v[j][i];
      }
    }
  }
#undef MC_LOADF
#pragma unroll
  for (int j = 0; j < kThinPx; ++j) {
    if (pix[j] >= a.P) continue;
#pragma unroll
    for (int m = 0; m < kThinM; ++m) {
      if (m >= a.M) break;
      const int c = g * a.M + m;
      const long idx = ybase[j] + static_cast<long>(c) * a.y_cstride;
      float v = acc[j][m];
      if (a.scale) v *= a.scale[c];
      if (a.shift) v += a.shift[c];
      if (a.residual) v += a.residual[idx];
      a.y[idx] = apply_act(v, a.act, a.slope);
    }
  }
}

// Packed filter wt[g][kt][m][kl] = w[g*wg_stride + wk_off[k] + m*wm_stride] with
// k = kt*16 + kl, zero where k >= K or m >= M.
__global__ void pack_weights_kernel(const float* __restrict__ w, float* __restrict__ wt,
                                    const int* __restrict__ wk_off, int G, int K, int Kpad,
                                    int M, int Mpad, int wm_stride, int wg_stride) {
  const long total = (long)G * Kpad * Mpad;
  const int KT = Kpad / BK;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total;
       i += (long)gridDim.x * blockDim.x) {
    const int kl = static_cast<int>(i % BK);
    long t = i / BK;
    const int m = static_cast<int>(t % Mpad);
    t /= Mpad;
    const int kt = static_cast<int>(t % KT);
    const int g = static_cast<int>(t / KT);
    const int k = kt * BK + kl;
    float v = 0.f;
    if (k < K && m < M) v = w[(long)g * wg_stride + wk_off[k] + (long)m * wm_stride];
    wt[i] = v;
  }
}

struct TileConfig {
  int bm, bn;
  int ks;  // 16-row K tiles per stage
  const char* name;
  void (*kernel[4])(const IgemmBatch);  // indexed by mode; [3] (pixel-quad pointwise) may be null
  void (*one_sub[4])(const IgemmBatch);  // the same for launches of one sub-problem, or null
};

const TileConfig kConfigs[] = {
    {128, 128, 1, "igemm_f32_128x128",
     {igemm_kernel<128, 128, 2, 2, 3, kModeMasks, 1>, igemm_kernel<128, 128, 2, 2, 3, kModeOneMask, 1>,
      igemm_kernel<128, 128, 2, 2, 3, kModePointwise, 1>}},
    {128, 64, 1, "igemm_f32_128x64",
     {igemm_kernel<128, 64, 2, 2, 4, kModeMasks, 1>, igemm_kernel<128, 64, 2, 2, 4, kModeOneMask, 1>,
      igemm_kernel<128, 64, 2, 2, 4, kModePointwise, 1>}},
    {64, 128, 1, "igemm_f32_64x128",
     {igemm_kernel<64, 128, 2, 2, 5, kModeMasks, 1>, igemm_kernel<64, 128, 2, 2, 5, kModeOneMask, 1>,
      igemm_kernel<64, 128, 2, 2, 5, kModePointwise, 1>}},
    {64, 64, 1, "igemm_f32_64x64",
     {igemm_kernel<64, 64, 2, 2, 8, kModeMasks, 1>, igemm_kernel<64, 64, 2, 2, 8, kModeOneMask, 1>,
      igemm_kernel<64, 64, 2, 2, 8, kModePointwise, 1>, igemm_kernel<64, 64, 2, 2, 8, kModePointwiseQuad, 1>},
     {igemm_kernel<64, 64, 2, 2, 8, kModeMasks, 1, true>, igemm_kernel<64, 64, 2, 2, 8, kModeOneMask, 1, true>,
      igemm_kernel<64, 64, 2, 2, 8, kModePointwise, 1, true>,
      igemm_kernel<64, 64, 2, 2, 8, kModePointwiseQuad, 1, true>}},
    {32, 128, 1, "igemm_f32_32x128",
     {igemm_kernel<32, 128, 1, 4, 4, kModeMasks, 1>, igemm_kernel<32, 128, 1, 4, 4, kModeOneMask, 1>,
      igemm_kernel<32, 128, 1, 4, 4, kModePointwise, 1>}},
    {32, 256, 1, "igemm_f32_32x256",
     {igemm_kernel<32, 256, 1, 4, 3, kModeMasks, 1>, igemm_kernel<32, 256, 1, 4, 3, kModeOneMask, 1>,
      igemm_kernel<32, 256, 1, 4, 3, kModePointwise, 1>}},
    {64, 256, 1, "igemm_f32_64x256",
     {igemm_kernel<64, 256, 1, 4, 2, kModeMasks, 1>, igemm_kernel<64, 256, 1, 4, 2, kModeOneMask, 1>,
      igemm_kernel<64, 256, 1, 4, 2, kModePointwise, 1>}},
    {64, 64, 2, "igemm_f32_64x64x32",
     {igemm_kernel<64, 64, 2, 2, 4, kModeMasks, 2>, igemm_kernel<64, 64, 2, 2, 4, kModeOneMask, 2>,
      igemm_kernel<64, 64, 2, 2, 4, kModePointwise, 2>}},
};
constexpr int kNumConfigs = sizeof(kConfigs) / sizeof(kConfigs[0]);

// One stride-1 gather problem: the whole Convolution, or one output-parity
// class of a Deconvolution.
struct SubProblem {
  int K = 0, Kpad = 0;
  int Hq = 0, Wq = 0;
  int q_sh = 1, q_sw = 1, in_oh = 0, in_ow = 0;
  int out_sh = 1, out_sw = 1, out_oh = 0, out_ow = 0;
  std::vector<int4> ktab;    // host copy: {byte offset, row-tap index, column-tap index, 0}
  std::vector<int> wk_off;   // host copy
  std::vector<int> tap_dh, tap_dw;  // bottom offset of each row / column tap index
  bool pointwise = false;    // every k is channel k at the pixel itself, always in range
  bool one_mask = false;     // at most 31 (row, column) tap pairs: one validity mask
  // The bottom descriptor starts tap_shift + pix_shift bytes before the blob:
  // tap offsets are stored plus tap_shift, pixel origins computed plus pix_shift,
  // so both are non-negative.
  int tap_shift = 0, pix_shift = 0;
  int* tap_dev = nullptr;    // tap_dh followed by tap_dw
  int4* ktab_dev = nullptr;
  int* wk_off_dev = nullptr;
  float* wt_dev = nullptr;
};

}  // namespace
}  // namespace mchip

using namespace mchip;

struct mcConvPlan {
  mcConvGeom geom;
  int Ho = 0, Wo = 0;
  int M = 0;        // output channels per group
  int Cin_g = 0;
  int Mpad = 0;
  int wm_stride = 0, wg_stride = 0;
  int forced_config = -1;
  int forced_split = 0;  // 0 = choose, >= 1 = this many K slices
  int forced_chunk = 0;  // 0 = as many images per launch as fit, else at most this many
  bool force_general = false;  // use the tap-table gather even for pointwise geometry
  // group == input channels: a direct kernel reads the layer's own filter layout
  bool depthwise = false;
  float* dw_weights = nullptr;  // copy of the [Cout, 1, kh, kw] filter blob
  // 3x3 stride 1: the Winograd path, and who decides (-1 = by size, 0 = never, 1 = always)
  WinogradState* winograd = nullptr;
  int winograd_mode = -1;
  std::vector<SubProblem> subs;
};

namespace {

// Optional per-launch timing: when enabled, every contraction launch is
// bracketed by HIP events on the stream it runs on.
struct TimedLaunch {
  hipEvent_t start, stop;
  double flops;   // algorithmic: what the layer's direct sum takes
  double issued;  // what the matrix pipe is given (less on the Winograd path)
  const char* name;
};
thread_local bool g_timing = false;
int g_winograd_default = -1;  // mode new plans start with
thread_local std::vector<TimedLaunch> g_timed;

// Tile choice.  With 256 CUs the tile count per CU is small for most layers, so
// load balance (the last, partly filled round of tiles) dominates: measured on
// ResNet-50 shapes the 64x64 tile, which runs 8 workgroups per CU, beats the
// larger tiles everywhere their extra reuse could matter.  Narrow outputs
// (<= 32 channels per group) use the 32-row tiles instead of padding M to 64.
int pick_config(const mcConvPlan* plan, long pixels) {
  if (plan->forced_config >= 0) return plan->forced_config;
  const int M = plan->M;
  int bm = 64, bn = 64;
  if (M <= 32) {
    bm = 32;
    const long tiles256 = (long)ceil_div(pixels, 256) * plan->geom.group;
    bn = tiles256 >= 8L * kNumCu ? 256 : 128;
  }
  for (int i = 0; i < kNumConfigs; ++i)
    if (kConfigs[i].bm == bm && kConfigs[i].bn == bn) return i;
  return 0;
}

// K slices for one launch.  A layer with few output tiles leaves most of the
// 8 workgroup slots per CU empty, and a lone workgroup pays the full global
// load latency on every K tile; slicing K brings the launch up to about one
// full round of workgroups, each slice still long enough to amortise its
// prologue and the summing of the slices.
// A handful of output channels over many pixels goes to the per-pixel kernel.
bool use_thin(const mcConvPlan* plan, int num) {
  long total_pixels = 0;
  for (const auto& s : plan->subs) total_pixels += (long)num * s.Hq * s.Wq;
  return plan->M <= kThinM && plan->forced_config < 0 && plan->forced_split == 0 &&
         total_pixels * plan->geom.group >= 65536;
}

int pick_split(const mcConvPlan* plan, long blocks, int KT) {
  if (plan->forced_split >= 1) return std::min(plan->forced_split, std::max(KT, 1));
  const long slots = 8L * kNumCu;
  if (blocks * 2 > slots) return 1;
  int s = static_cast<int>(slots / blocks);
  s = std::min(s, KT / 8);
  // A launch of a few dozen workgroups (detection heads on small maps) is pure
  // latency: its time is the number of K tiles per slice, so it takes finer slices.
  // Below one workgroup per CU the launch still gains from finer slices than a
  // fuller one (1024->150 3x3 on 8x19x19: 128 us with 8 slices, 98 us with 12).
  s = std::min(s, blocks * 10 <= kNumCu ? 24 : (blocks < kNumCu ? 16 : 8));
  return std::max(s, 1);
}

int free_sub(SubProblem& s) {
  if (s.ktab_dev) (void)hipFree(s.ktab_dev);
  if (s.tap_dev) (void)hipFree(s.tap_dev);
  s.tap_dev = nullptr;
  if (s.wk_off_dev) (void)hipFree(s.wk_off_dev);
  if (s.wt_dev) (void)hipFree(s.wt_dev);
  s.ktab_dev = nullptr;
  s.wk_off_dev = nullptr;
  s.wt_dev = nullptr;
  return 0;
}

// floor division for possibly negative numerators
inline int floordiv(int a, int b) { return (a >= 0) ? a / b : -((-a + b - 1) / b); }

}  // namespace

extern "C" {

int mcConvPlanCreate(const mcConvGeom* gp, mcConvPlan** out) {
  MC_REQUIRE(gp && out, "mcConvPlanCreate: null argument");
  const mcConvGeom& g = *gp;
  MC_REQUIRE(g.channels_in > 0 && g.channels_out > 0 && g.height_in > 0 && g.width_in > 0,
             "mcConvPlanCreate: non-positive blob dimension");
  MC_REQUIRE(g.kernel_h > 0 && g.kernel_w > 0, "Filter dimensions must be nonzero.");
  MC_REQUIRE(g.stride_h > 0 && g.stride_w > 0, "Stride dimensions must be nonzero.");
  MC_REQUIRE(g.dilation_h > 0 && g.dilation_w > 0, "Dilation dimensions must be nonzero.");
  MC_REQUIRE(g.pad_h >= 0 && g.pad_w >= 0, "Padding must be non-negative.");
  MC_REQUIRE(g.group > 0 && g.channels_in % g.group == 0 && g.channels_out % g.group == 0,
             "Number of channels and of outputs must be multiples of group.");
  MC_REQUIRE(g.height_in < 16384 && g.width_in < 16384 && g.kernel_h * g.dilation_h < 16384 &&
                 g.kernel_w * g.dilation_w < 16384,
             "mcConvPlanCreate: spatial extent too large for the tap table");

  mcConvPlan* plan = new mcConvPlan();
  plan->geom = g;
  const int ext_h = g.dilation_h * (g.kernel_h - 1) + 1;
  const int ext_w = g.dilation_w * (g.kernel_w - 1) + 1;
  if (!g.transposed) {
    plan->Ho = (g.height_in + 2 * g.pad_h - ext_h) / g.stride_h + 1;
    plan->Wo = (g.width_in + 2 * g.pad_w - ext_w) / g.stride_w + 1;
  } else {
    plan->Ho = g.stride_h * (g.height_in - 1) + ext_h - 2 * g.pad_h;
    plan->Wo = g.stride_w * (g.width_in - 1) + ext_w - 2 * g.pad_w;
  }
  if (plan->Ho <= 0 || plan->Wo <= 0) {
    const int ho = plan->Ho, wo = plan->Wo;
    delete plan;
    return fail("mcConvPlanCreate: empty output (%d x %d)", ho, wo);
  }
  plan->M = g.channels_out / g.group;
  plan->Cin_g = g.channels_in / g.group;
  if (!g.transposed && g.group > 1 && g.group == g.channels_in) {
    plan->depthwise = true;
    const hipError_t e =
        hipMalloc(&plan->dw_weights, sizeof(float) * (size_t)g.channels_out * g.kernel_h * g.kernel_w);
    if (e != hipSuccess) {
      delete plan;
      return fail("mcConvPlanCreate: device set-up failed: %s", hipGetErrorString(e));
    }
    *out = plan;
    return 0;
  }
  plan->Mpad = ceil_div(plan->M, 128) * 128;
  const int HW = g.height_in * g.width_in;
  const int khkw = g.kernel_h * g.kernel_w;

  if (!g.transposed) {
    SubProblem s;
    s.K = plan->Cin_g * khkw;
    s.Hq = plan->Ho;
    s.Wq = plan->Wo;
    s.q_sh = g.stride_h;
    s.q_sw = g.stride_w;
    s.in_oh = -g.pad_h;
    s.in_ow = -g.pad_w;
    for (int i = 0; i < g.kernel_h; ++i) s.tap_dh.push_back(i * g.dilation_h);
    for (int j = 0; j < g.kernel_w; ++j) s.tap_dw.push_back(j * g.dilation_w);
    for (int c = 0; c < plan->Cin_g; ++c)
      for (int i = 0; i < g.kernel_h; ++i)
        for (int j = 0; j < g.kernel_w; ++j) {
          const int dh = i * g.dilation_h, dw = j * g.dilation_w;
          s.ktab.push_back(make_int4((c * HW + dh * g.width_in + dw) * 4, i, j, i * g.kernel_w + j));
          s.wk_off.push_back((c * g.kernel_h + i) * g.kernel_w + j);
        }
    s.pointwise = g.kernel_h == 1 && g.kernel_w == 1 && g.pad_h == 0 && g.pad_w == 0;
    plan->wm_stride = s.K;
    plan->wg_stride = plan->M * s.K;
    plan->subs.push_back(std::move(s));
  } else {
    plan->wm_stride = khkw;
    plan->wg_stride = plan->Cin_g * plan->M * khkw;
    for (int rh = 0; rh < g.stride_h; ++rh)
      for (int rw = 0; rw < g.stride_w; ++rw) {
        if (rh >= plan->Ho || rw >= plan->Wo) continue;
        SubProblem s;
        s.Hq = (plan->Ho - rh + g.stride_h - 1) / g.stride_h;
        s.Wq = (plan->Wo - rw + g.stride_w - 1) / g.stride_w;
        s.out_sh = g.stride_h;
        s.out_sw = g.stride_w;
        s.out_oh = rh;
        s.out_ow = rw;
        // top row oh = s*q + rh receives bottom row ih with oh = ih*s - p + kh*d,
        // i.e. ih = q + (rh + p - kh*d)/s whenever that quotient is exact.
        std::vector<int> tap_h, off_h, tap_w, off_w;
        for (int i = 0; i < g.kernel_h; ++i) {
          const int num = rh + g.pad_h - i * g.dilation_h;
          if (((num % g.stride_h) + g.stride_h) % g.stride_h == 0) {
            tap_h.push_back(i);
            off_h.push_back(floordiv(num, g.stride_h));
          }
        }
        for (int j = 0; j < g.kernel_w; ++j) {
          const int num = rw + g.pad_w - j * g.dilation_w;
          if (((num % g.stride_w) + g.stride_w) % g.stride_w == 0) {
            tap_w.push_back(j);
            off_w.push_back(floordiv(num, g.stride_w));
          }
        }
        for (int c = 0; c < plan->Cin_g; ++c)
          for (size_t i = 0; i < tap_h.size(); ++i)
            for (size_t j = 0; j < tap_w.size(); ++j) {
              s.ktab.push_back(make_int4((c * HW + off_h[i] * g.width_in + off_w[j]) * 4,
                                         static_cast<int>(i), static_cast<int>(j),
                                         static_cast<int>(i * tap_w.size() + j)));
              s.wk_off.push_back(c * plan->M * khkw + tap_h[i] * g.kernel_w + tap_w[j]);
            }
        s.tap_dh = off_h;
        s.tap_dw = off_w;
        s.K = static_cast<int>(s.ktab.size());
        plan->subs.push_back(std::move(s));
      }
  }

  for (auto& s : plan->subs) {
    s.Kpad = ceil_div(s.K, 2 * BK) * 2 * BK;  // whole stages for every configuration
    // Padding rows multiply zero weights; row-tap index 31 is out of the image
    // for every pixel, so nothing is fetched for them.
    while (static_cast<int>(s.ktab.size()) < s.Kpad) s.ktab.push_back(make_int4(0, 31, 0, 31));
    int min_tap = 0;
    for (const int4& t : s.ktab) min_tap = std::min(min_tap, t.x);
    s.tap_shift = -min_tap;
    for (int4& t : s.ktab) t.x += s.tap_shift;
    s.pix_shift = std::max(0, -(s.in_oh * g.width_in + s.in_ow) * 4);
    if (s.Kpad == 0) continue;
    const size_t wt_bytes = sizeof(float) * (size_t)g.group * s.Kpad * plan->Mpad;
    hipError_t e = hipSuccess;
    const char* what = nullptr;
    // Few taps and channels in fours: reorder the K rows from (channel, tap) to
    // (channel block of 4, tap, channel in block).  Any order is a valid GEMM as
    // long as filter packing (wk_off) follows it; this one gives a thread's four
    // rows per step a common tap while the taps of a channel stay close in K, so
    // their overlapping input lines are still re-read from L1.
    const int pairs = static_cast<int>(s.tap_dh.size() * s.tap_dw.size());
    s.one_mask = pairs >= 1 && pairs <= 31 && plan->Cin_g % 4 == 0 && s.K == plan->Cin_g * pairs;
    if (s.one_mask) {
      std::vector<int4> kt(s.K);
      std::vector<int> wk(s.K);
      int k = 0;
      for (int cb = 0; cb < plan->Cin_g / 4; ++cb)
        for (int t = 0; t < pairs; ++t)
          for (int ci = 0; ci < 4; ++ci, ++k) {
            const int old = (cb * 4 + ci) * pairs + t;
            kt[k] = s.ktab[old];
            wk[k] = s.wk_off[old];
          }
      std::copy(kt.begin(), kt.end(), s.ktab.begin());
      s.wk_off = wk;
    }
    if (s.tap_dh.size() > 31 || s.tap_dw.size() > 31)
      what = "kernels with more than 31 taps per dimension are not supported";
    else if (wt_bytes >= (1ull << 31))
      what = "packed filter exceeds 2 GiB";
    if (!what) {
      std::vector<int> taps(s.tap_dh);
      taps.insert(taps.end(), s.tap_dw.begin(), s.tap_dw.end());
      taps.push_back(0);  // never empty
      e = hipMalloc(&s.ktab_dev, sizeof(int4) * s.Kpad);
      if (e == hipSuccess) e = hipMalloc(&s.wk_off_dev, sizeof(int) * s.K);
      if (e == hipSuccess) e = hipMalloc(&s.tap_dev, sizeof(int) * taps.size());
      if (e == hipSuccess) e = hipMalloc(&s.wt_dev, wt_bytes);
      if (e == hipSuccess)
        e = hipMemcpy(s.ktab_dev, s.ktab.data(), sizeof(int4) * s.Kpad, hipMemcpyHostToDevice);
      if (e == hipSuccess)
        e = hipMemcpy(s.wk_off_dev, s.wk_off.data(), sizeof(int) * s.K, hipMemcpyHostToDevice);
      if (e == hipSuccess)
        e = hipMemcpy(s.tap_dev, taps.data(), sizeof(int) * taps.size(), hipMemcpyHostToDevice);
    }
    if (what || e != hipSuccess) {
      for (auto& t : plan->subs) free_sub(t);
      delete plan;
      return what ? fail("mcConvPlanCreate: %s", what)
                  : fail("mcConvPlanCreate: device set-up failed: %s", hipGetErrorString(e));
    }
  }
  plan->winograd = winograd_create(g, plan->Ho, plan->Wo);
  plan->winograd_mode = g_winograd_default;
  *out = plan;
  return 0;
}

int mcInnerProductPlanCreate(int K, int N, int transpose, mcConvPlan** out) {
  MC_REQUIRE(K > 0 && N > 0 && out, "mcInnerProductPlanCreate: bad argument");
  mcConvGeom g = {K, 1, 1, N, 1, 1, 1, 1, 0, 0, 1, 1, 1, 0};
  if (mcConvPlanCreate(&g, out)) return -1;
  if (transpose) {
    // weights are K x N: element (k, m) sits at k*N + m
    mcConvPlan* plan = *out;
    SubProblem& s = plan->subs[0];
    for (int k = 0; k < s.K; ++k) s.wk_off[k] = k * N;
    plan->wm_stride = 1;
    hipError_t e =
        hipMemcpy(s.wk_off_dev, s.wk_off.data(), sizeof(int) * s.K, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
      mcConvPlanDestroy(plan);
      *out = nullptr;
      return fail("mcInnerProductPlanCreate: %s", hipGetErrorString(e));
    }
  }
  return 0;
}

int mcConvPlanDestroy(mcConvPlan* plan) {
  if (!plan) return 0;
  if (plan->dw_weights) (void)hipFree(plan->dw_weights);
  winograd_destroy(plan->winograd);
  for (auto& s : plan->subs) free_sub(s);
  delete plan;
  return 0;
}

int mcConvPlanOutputShape(const mcConvPlan* plan, int* ho, int* wo) {
  MC_REQUIRE(plan, "mcConvPlanOutputShape: null plan");
  if (ho) *ho = plan->Ho;
  if (wo) *wo = plan->Wo;
  return 0;
}

int mcConvPlanSetWeights(mcConvPlan* plan, const float* weights, void* stream) {
  MC_REQUIRE(plan && weights, "mcConvPlanSetWeights: null argument");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (plan->depthwise) {
    const mcConvGeom& g = plan->geom;
    MC_HIP(hipMemcpyAsync(plan->dw_weights, weights,
                          sizeof(float) * (size_t)g.channels_out * g.kernel_h * g.kernel_w,
                          hipMemcpyDeviceToDevice, st));
    return 0;
  }
  for (auto& s : plan->subs) {
    if (s.Kpad == 0) continue;
    const long total = (long)plan->geom.group * s.Kpad * plan->Mpad;
    pack_weights_kernel<<<ew_blocks(total, 256), 256, 0, st>>>(
        weights, s.wt_dev, s.wk_off_dev, plan->geom.group, s.K, s.Kpad, plan->M, plan->Mpad,
        plan->wm_stride, plan->wg_stride);
    MC_LAUNCH_CHECK();
  }
  if (plan->winograd && winograd_set_weights(plan->winograd, weights, st)) return -1;
  return 0;
}

int mcConvPlanForceWinograd(mcConvPlan* plan, int mode) {
  MC_REQUIRE(plan && mode >= -1 && mode <= 1, "mcConvPlanForceWinograd: bad argument");
  MC_REQUIRE(mode != 1 || plan->winograd,
             "mcConvPlanForceWinograd: not a 3x3 stride-1 convolution of one group");
  plan->winograd_mode = mode;
  return 0;
}

int mcConvWinogradDefault(int mode) {
  MC_REQUIRE(mode >= -1 && mode <= 1, "mcConvWinogradDefault: bad argument");
  g_winograd_default = mode;
  return 0;
}

int mcConvPlanForceConfig(mcConvPlan* plan, int config) {
  MC_REQUIRE(plan, "mcConvPlanForceConfig: null plan");
  // config + 100 pins the same tile with the two-mask tap-table gather (tests
  // compare the pointwise and one-mask fast paths against it)
  plan->force_general = config >= 100;
  if (config >= 100) config -= 100;
  MC_REQUIRE(config >= -1 && config < kNumConfigs, "mcConvPlanForceConfig: no such configuration");
  plan->forced_config = config;
  return 0;
}

int mcConvPlanForceChunk(mcConvPlan* plan, int images) {
  MC_REQUIRE(plan && images >= 0, "mcConvPlanForceChunk: bad argument");
  plan->forced_chunk = images;
  return 0;
}

int mcConvPlanForceSplit(mcConvPlan* plan, int slices) {
  MC_REQUIRE(plan, "mcConvPlanForceSplit: null plan");
  MC_REQUIRE(slices >= 0 && slices <= 64, "mcConvPlanForceSplit: slices out of range");
  plan->forced_split = slices;
  return 0;
}

}  // extern "C"

namespace {

// top_second != nullptr: the plan's output channels [0, c_first) go to `top`, the
// others to top_second.
// One launch (plus, for two tops, the pass that sums K slices) over `num` images that fit the
// kernels' 31-bit byte offsets; conv_forward() cuts larger batches into such runs.
int conv_forward_images(const mcConvPlan* plan, int num, const float* bottom, float* top,
                        const mcEpilogue* ep, void* stream, float* top_second, int c_first) {
  const mcConvGeom& g = plan->geom;
  const long in_count = (long)num * g.channels_in * g.height_in * g.width_in;
  const long out_count = (long)num * g.channels_out * plan->Ho * plan->Wo;
  // the blobs are addressed through 31-bit byte offsets
  MC_REQUIRE(plan->depthwise || (in_count < (1L << 29) && out_count < (1L << 29)),
             "mcConvForward: image run exceeds 2^29 elements");
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* const top_first = top;
  if (top_second) {
    MC_REQUIRE(!plan->depthwise && g.group == 1 && c_first > 0 && c_first < g.channels_out &&
                   !(ep && ep->residual),
               "mcConvForwardTwoTops: needs group 1, a split inside the output channels and no "
               "residual");
  }
  if (plan->depthwise) {
    DepthwiseArgs d = {bottom, plan->dw_weights, top, ep ? ep->scale : nullptr,
                       ep ? ep->shift : nullptr, ep ? ep->residual : nullptr, num,
                       g.channels_in, plan->M, g.height_in, g.width_in, plan->Ho, plan->Wo,
                       g.kernel_h, g.kernel_w, g.stride_h, g.stride_w, g.pad_h, g.pad_w,
                       g.dilation_h, g.dilation_w, ep ? ep->activation : MC_ACT_NONE,
                       ep ? ep->negative_slope : 0.f};
    TimedLaunch tl;
    if (g_timing) {
      MC_HIP(hipEventCreate(&tl.start));
      MC_HIP(hipEventCreate(&tl.stop));
      tl.flops = tl.issued = mcConvPlanFlops(plan, num);
      tl.name = "depthwise_f32";
      MC_HIP(hipEventRecord(tl.start, st));
    }
    if (depthwise_forward(d, st)) return -1;
    if (g_timing) {
      MC_HIP(hipEventRecord(tl.stop, st));
      g_timed.push_back(tl);
    }
    return 0;
  }

  // Sub-problems that have pixels at this batch size, their tile configuration
  // (one for the whole plan: the largest sub-problem decides) and K slices.
  std::vector<const SubProblem*> live;
  long max_pixels = 0;
  for (const auto& s : plan->subs) {
    const long pixels = (long)num * s.Hq * s.Wq;
    if (pixels == 0) continue;
    MC_REQUIRE(pixels < (1L << 31), "mcConvForward: too many output pixels");
    live.push_back(&s);
    max_pixels = std::max(max_pixels, pixels);
  }
  if (live.empty()) return 0;
  const TileConfig& cfg = kConfigs[pick_config(plan, max_pixels)];
  const int MT = ceil_div(plan->M, cfg.bm);
  long total_blocks = 0;
  int min_kt = 1 << 30;
  bool pointwise = !plan->force_general, one_mask = !plan->force_general;
  bool quad_ok = true;  // stride-1 pointwise on planes of a multiple of four pixels, K a multiple of 16
  double flops = 0.;
  for (const SubProblem* s : live) {
    const long pixels = (long)num * s->Hq * s->Wq;
    total_blocks += (long)MT * ceil_div(pixels, cfg.bn) * g.group;
    if (s->Kpad > 0) min_kt = std::min(min_kt, s->Kpad / (BK * cfg.ks));
    pointwise = pointwise && s->pointwise;
    quad_ok = quad_ok && s->q_sh == 1 && s->q_sw == 1 && s->Hq == g.height_in && s->Wq == g.width_in &&
              (s->Hq * s->Wq) % 4 == 0 && s->K % 16 == 0 && s->in_oh == 0 && s->in_ow == 0 &&
              // ... and pixel p of an image is element p of its top plane as well (the kernel
              // then needs no row / column of a pixel on either side)
              s->out_sh == 1 && s->out_sw == 1 && s->out_oh == 0 && s->out_ow == 0 && s->Hq == plan->Ho &&
              s->Wq == plan->Wo;
    one_mask = one_mask && s->one_mask;
    flops += 2.0 * pixels * plan->M * g.group * s->K;
  }
  if (min_kt == (1 << 30)) min_kt = 1;
  // (the per-pixel kernel writes one top only)
  const bool thin = !top_second && use_thin(plan, num);
  // slices are chosen for the plan as a whole: all sub-problems of a launch run
  // side by side
  // Two tops are told apart by the pass that sums the slices, so such a launch
  // has at least two of them (a slice past the last K tile adds zeros).
  int slices = thin ? 1 : pick_split(plan, total_blocks, min_kt);
  if (top_second && slices == 1) slices = 2;
  const long slice_stride = (out_count + 3) / 4 * 4;
  float* ws = nullptr;
  // One top: the slices are summed inside the launch by the last workgroup of each
  // tile.  Two tops: a pass of its own sums them and tells the tops apart.
  const bool sum_in_launch = slices > 1 && !top_second;
  int* counters = nullptr;
  long partial_tiles = 0;
  if (sum_in_launch) {
    for (size_t first = 0; first < live.size(); first += kMaxSubs) {
      const size_t nsub = std::min<size_t>(kMaxSubs, live.size() - first);
      long most = 0;
      for (size_t i = 0; i < nsub; ++i)
        most = std::max<long>(most, (long)MT * ceil_div((long)num * live[first + i]->Hq * live[first + i]->Wq,
                                                         cfg.bn));
      partial_tiles = std::max<long>(partial_tiles, most * g.group * (long)nsub);
    }
    MC_REQUIRE(partial_tiles < (1L << 31), "mcConvForward: grid too large");
    if (stream_workspace(st, sizeof(float) * partial_tiles * cfg.bm * cfg.bn * slices, &ws)) return -1;
    if (stream_counters(st, static_cast<size_t>(partial_tiles), &counters)) return -1;
  } else if (slices > 1) {
    if (stream_workspace(st, sizeof(float) * slice_stride * slices, &ws)) return -1;
  }

  TimedLaunch tl;
  const bool timed = g_timing;
  if (timed) {
    MC_HIP(hipEventCreate(&tl.start));
    MC_HIP(hipEventCreate(&tl.stop));
    tl.flops = tl.issued = flops;
    tl.name = thin ? "thin_f32" : cfg.name;
    MC_HIP(hipEventRecord(tl.start, st));
  }
  for (size_t first = 0; first < live.size(); first += kMaxSubs) {
    const int nsub = static_cast<int>(std::min<size_t>(kMaxSubs, live.size() - first));
    IgemmBatch batch;
    std::memset(&batch, 0, sizeof(batch));
    batch.slices = slices;
    long max_blocks = 0;
    for (int i = 0; i < nsub; ++i) {
      const SubProblem& s = *live[first + i];
      const long pixels = (long)num * s.Hq * s.Wq;
      IgemmArgs& a = batch.sub[i];
      a.wt = s.wt_dev;
      a.y = top;
      a.ktab = s.ktab_dev;
      a.tap_dh = s.tap_dev;
      a.tap_dw = s.tap_dev + s.tap_dh.size();
      // a sub-problem without taps (K == 0) has no tables on the device
      a.n_dh = s.tap_dev ? static_cast<int>(s.tap_dh.size()) : 0;
      a.n_dw = s.tap_dev ? static_cast<int>(s.tap_dw.size()) : 0;
      const long shift = (long)s.tap_shift + s.pix_shift;
      MC_REQUIRE(in_count * 4 + 2 * shift + 64 < (1L << 31),
                 "mcConvForward: bottom blob too large for 31-bit byte offsets");
      a.x = reinterpret_cast<const float*>(reinterpret_cast<const char*>(bottom) - shift);
      a.x_bytes = static_cast<unsigned>(in_count * 4 + shift);
      a.pix_shift = s.pix_shift;
      a.wt_bytes = static_cast<unsigned>(sizeof(float) * (size_t)g.group * s.Kpad * plan->Mpad);
      a.K = s.K;
      a.x_cstride = g.height_in * g.width_in;
      a.scale = ep ? ep->scale : nullptr;
      a.shift = ep ? ep->shift : nullptr;
      a.residual = ep ? ep->residual : nullptr;
      a.P = static_cast<int>(pixels);
      a.Hq = s.Hq;
      a.Wq = s.Wq;
      a.HqWq = s.Hq * s.Wq;
      // columns up to the end of the last pixel tile are divided (and then ignored)
      make_fast_div(a.HqWq, pixels + 512, &a.div_hw_mul, &a.div_hw_shift);
      make_fast_div(a.Wq, (unsigned long long)a.HqWq + 1, &a.div_w_mul, &a.div_w_shift);
      a.y_bytes = static_cast<unsigned>(out_count * 4);
      a.c_bytes = static_cast<unsigned>(g.channels_out) * 4;
      a.H = g.height_in;
      a.W = g.width_in;
      a.q_sh = s.q_sh;
      a.q_sw = s.q_sw;
      a.in_oh = s.in_oh;
      a.in_ow = s.in_ow;
      a.x_nstride = g.channels_in * g.height_in * g.width_in;
      a.x_gstride = plan->Cin_g * g.height_in * g.width_in;
      a.M = plan->M;
      a.Mpad = plan->Mpad;
      a.Kpad = s.Kpad;
      a.Wo = plan->Wo;
      a.y_cstride = plan->Ho * plan->Wo;
      a.y_nstride = g.channels_out * plan->Ho * plan->Wo;
      a.out_sh = s.out_sh;
      a.out_sw = s.out_sw;
      a.out_oh = s.out_oh;
      a.out_ow = s.out_ow;
      a.MT = MT;
      a.NT = ceil_div(pixels, cfg.bn);
      make_fast_div(a.MT, (unsigned long long)a.MT * a.NT + 1, &a.div_mt_mul, &a.div_mt_shift);
      a.act = ep ? ep->activation : MC_ACT_NONE;
      a.slope = ep ? ep->negative_slope : 0.f;
      const long blocks = (long)a.MT * a.NT;
      MC_REQUIRE(blocks < (1L << 31), "mcConvForward: grid too large");
      max_blocks = std::max(max_blocks, blocks);
      // every slice gets the same number of K tiles; slices past the last tile
      // of a short sub-problem write zeros
      a.kt_per_split = ceil_div(std::max(s.Kpad / (BK * cfg.ks), 1), slices);
      a.split_stride = 0;
      a.partial = nullptr;
      a.counters = nullptr;
      a.partial_tiles = 0;
      if (sum_in_launch) {
        a.partial = ws;
        a.counters = counters;
        a.partial_tiles = static_cast<int>(partial_tiles);
      } else if (slices > 1) {
        a.y = ws;
        a.split_stride = static_cast<int>(slice_stride);
        a.scale = a.shift = a.residual = nullptr;
        a.act = MC_ACT_NONE;
      }
    }
    if (thin) {
      long most = 0;
      for (int i = 0; i < nsub; ++i) most = std::max<long>(most, batch.sub[i].P);
      dim3 grid(static_cast<unsigned>(ceil_div(most, 256L * kThinPx)), g.group, nsub);
      thin_conv_kernel<<<grid, 256, 0, st>>>(batch, pointwise ? 1 : 0);
    } else {
      dim3 grid(static_cast<unsigned>(max_blocks), g.group, nsub * slices);
      // A launch with less than one round of workgroups asks for enough LDS that
      // at most ceil(workgroups / CUs) of them fit a CU: the dispatcher then cannot
      // fill some CUs to eight and leave others short (1-3 % on such launches).
      unsigned extra_lds = 0;
      const long wgs = max_blocks * g.group * nsub * slices;
      if (wgs < 8L * kNumCu) {
        const int limit = std::max<long>(3, ceil_div(wgs, static_cast<long>(kNumCu)));
        const long stat = 2L * cfg.ks * (cfg.bm + cfg.bn) * LDK * 4;
        const long want = (160L * 1024 / limit) / 1024 * 1024;
        if (limit < 8 && want > stat) extra_lds = static_cast<unsigned>(want - stat);
      }
      int mode = pointwise ? kModePointwise : (one_mask ? kModeOneMask : kModeMasks);
      if (pointwise && quad_ok && cfg.kernel[kModePointwiseQuad]) mode = kModePointwiseQuad;
      auto kernel = (nsub == 1 && cfg.one_sub[mode]) ? cfg.one_sub[mode] : cfg.kernel[mode];
      kernel<<<grid, 256, extra_lds, st>>>(batch);
    }
    MC_LAUNCH_CHECK();
  }
  if (slices > 1 && top_second) {
    splitk_reduce_two_kernel<<<static_cast<unsigned>(ceil_div(out_count, 256L)), 256, 0, st>>>(
        ws, slices, slice_stride, out_count, top_first, top_second, c_first, ep ? ep->scale : nullptr,
        ep ? ep->shift : nullptr, plan->Ho * plan->Wo, g.channels_out,
        ep ? ep->activation : MC_ACT_NONE, ep ? ep->negative_slope : 0.f);
    MC_LAUNCH_CHECK();
  }
  if (timed) {
    MC_HIP(hipEventRecord(tl.stop, st));
    g_timed.push_back(tl);
  }
  return 0;
}

// Whether a call with `num` images runs on the Winograd path.
bool takes_winograd(const mcConvPlan* plan, int num) {
  return plan->winograd && plan->winograd_mode != 0 && plan->forced_config < 0 &&
         winograd_fits(plan->winograd, num) &&
         (plan->winograd_mode == 1 || winograd_pays(plan->winograd, num));
}

// The reference convolves image by image and so takes any blob an int can count
// (base_conv_layer.cpp:254-271).  Here a launch covers as many images as the 31-bit
// byte offsets of the buffer descriptors allow (fewer than 2^29 elements in the
// bottom and in the top run, offset shifts included); a larger batch is cut into
// equal runs of whole images, each with its own launch, epilogue and residual rows.
int conv_forward(const mcConvPlan* plan, int num, const float* bottom, float* top,
                 const mcEpilogue* ep, void* stream, float* top_second, int c_first) {
  MC_REQUIRE(plan && bottom && top, "mcConvForward: null argument");
  MC_REQUIRE(num > 0, "mcConvForward: batch must be positive");
  const mcConvGeom& g = plan->geom;
  if (plan->depthwise)  // indexed with 64-bit integers throughout
    return conv_forward_images(plan, num, bottom, top, ep, stream, top_second, c_first);
  if (takes_winograd(plan, num)) {
    TimedLaunch tl;
    const bool timed = g_timing;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (timed) {
      MC_HIP(hipEventCreate(&tl.start));
      MC_HIP(hipEventCreate(&tl.stop));
      tl.flops = mcConvPlanFlops(plan, num);
      tl.issued = winograd_issued_flops(plan->winograd, num);
      tl.name = "winograd_f32";
      MC_HIP(hipEventRecord(tl.start, st));
    }
    const int rc = winograd_forward(plan->winograd, num, bottom, top, ep, stream, top_second, c_first,
                                    plan->forced_chunk, plan->forced_split);
    if (timed) {
      MC_HIP(hipEventRecord(tl.stop, st));
      g_timed.push_back(tl);
    }
    return rc;
  }
  const long in_img = (long)g.channels_in * g.height_in * g.width_in;
  const long out_img = (long)g.channels_out * plan->Ho * plan->Wo;
  long shift = 0;
  for (const auto& s : plan->subs) shift = std::max(shift, (long)s.tap_shift + s.pix_shift);
  const long lim = (1L << 29) - 1;
  long per = std::min(lim / in_img, lim / out_img);
  per = std::min(per, ((1L << 31) - 65 - 2 * shift) / (4 * in_img));
  if (plan->forced_chunk > 0) per = std::min<long>(per, plan->forced_chunk);
  MC_REQUIRE(per >= 1, "mcConvForward: a single image exceeds 2^29 elements");
  if (num <= per)
    return conv_forward_images(plan, num, bottom, top, ep, stream, top_second, c_first);
  const int runs = ceil_div(num, per);
  const int run_len = ceil_div(num, runs);
  const long hw_out = (long)plan->Ho * plan->Wo;
  const long first_img = top_second ? c_first * hw_out : out_img;
  const long second_img = out_img - first_img;
  for (int n0 = 0; n0 < num; n0 += run_len) {
    const int n = std::min(run_len, num - n0);
    mcEpilogue run_ep;
    if (ep) {
      run_ep = *ep;
      if (ep->residual) run_ep.residual = ep->residual + n0 * out_img;
    }
    if (conv_forward_images(plan, n, bottom + n0 * in_img, top + n0 * first_img,
                            ep ? &run_ep : nullptr, stream,
                            top_second ? top_second + n0 * second_img : nullptr, c_first))
      return -1;
  }
  return 0;
}

}  // namespace

extern "C" {

int mcConvForward(const mcConvPlan* plan, int num, const float* bottom, float* top,
                  const mcEpilogue* ep, void* stream) {
  return conv_forward(plan, num, bottom, top, ep, stream, nullptr, 0);
}

int mcConvForwardTwoTops(const mcConvPlan* plan, int num, const float* bottom, float* top_first,
                         int channels_first, float* top_second, const mcEpilogue* ep,
                         void* stream) {
  MC_REQUIRE(top_second, "mcConvForwardTwoTops: null argument");
  return conv_forward(plan, num, bottom, top_first, ep, stream, top_second, channels_first);
}

int mcConvTimingEnable(int on) {
  g_timing = on != 0;
  return 0;
}

int mcConvTimingCollectDetail(double* total_ms, long* launches, double* flops, double* issued_flops,
                              long* winograd) {
  double ms = 0., fl = 0., is = 0.;
  long wino = 0;
  for (auto& t : g_timed) {
    MC_HIP(hipEventSynchronize(t.stop));
    float e = 0.f;
    MC_HIP(hipEventElapsedTime(&e, t.start, t.stop));
    ms += e;
    fl += t.flops;
    is += t.issued;
    wino += t.issued != t.flops;
    (void)hipEventDestroy(t.start);
    (void)hipEventDestroy(t.stop);
  }
  if (total_ms) *total_ms = ms;
  if (launches) *launches = static_cast<long>(g_timed.size());
  if (flops) *flops = fl;
  if (issued_flops) *issued_flops = is;
  if (winograd) *winograd = wino;
  g_timed.clear();
  return 0;
}

int mcConvTimingCollect(double* total_ms, long* launches, double* flops) {
  return mcConvTimingCollectDetail(total_ms, launches, flops, nullptr, nullptr);
}

double mcConvPlanFlops(const mcConvPlan* plan, int num) {
  if (!plan) return 0.;
  const mcConvGeom& g = plan->geom;
  const double taps = (double)g.kernel_h * g.kernel_w;
  if (!g.transposed)
    return 2. * num * g.channels_out * plan->Ho * plan->Wo * (g.channels_in / g.group) * taps;
  return 2. * num * g.channels_in * g.height_in * g.width_in * (g.channels_out / g.group) * taps;
}

const char* mcConvPlanKernelName(const mcConvPlan* plan, int num) {
  if (plan && plan->depthwise) return "depthwise_f32";
  if (!plan || plan->subs.empty()) return "";
  if (takes_winograd(plan, num)) return "winograd_f32";
  if (use_thin(plan, num)) return "thin_f32";
  const auto& s = plan->subs[0];
  return kConfigs[pick_config(plan, (long)num * s.Hq * s.Wq)].name;
}

}  // extern "C"
