// SSD DetectionOutput on the device: box decode, per-(image, class) candidate
// ordering + greedy NMS, per-image keep_top_k, row emission.
//
// Restates DetectionOutputLayer::Forward_cpu (reference
// src/layers/detection_output_layer.cpp:74-226) with the helpers of
// src/util/bbox_util.cpp (DecodeBBox :242-330, GetMaxScoreIndex :523-540,
// JaccardOverlap :184-204, ApplyNMSFast :681-716).  The reference's device path
// (detection_output_layer.cu:14-152) decodes on the GPU and then runs the whole
// selection on the host; here nothing but the final row count returns to the
// host.
//
// Compiled with -ffp-contract=off so that decoded coordinates, overlaps and
// therefore the kept indices equal the CPU path's bit for bit.
#include "../mc_common.h"
#include "block_sort.h"
#include "mchip/kernels.h"

namespace mchip {
namespace {

struct DBox {
  float xmin, ymin, xmax, ymax, size;
};

__device__ __forceinline__ float dbox_size(float xmin, float ymin, float xmax, float ymax) {
  if (xmax < xmin || ymax < ymin) return 0.f;
  const float width = xmax - xmin;
  const float height = ymax - ymin;
  return width * height;
}

// One thread per (image, loc class, prior).  code_type 1 CORNER, 2 CENTER_SIZE,
// 3 CORNER_SIZE.  exp() and the "/ 2." halvings are evaluated in double, as the
// reference's expressions promote.
__global__ __launch_bounds__(256) void det_decode_kernel(
    const float* __restrict__ loc, const float* __restrict__ prior, int num, int P,
    int loc_classes, int code_type, int var_in_target, DBox* __restrict__ out,
    int* __restrict__ cut_tie_flag, const float* __restrict__ conf, int C,
    uint32_t* __restrict__ keys_by_class) {
  const long total = (long)num * loc_classes * P;
  const long t = blockIdx.x * 256L + threadIdx.x;
  if (t == 0 && cut_tie_flag) *cut_tie_flag = 0;  // raised by det_select_kernel, two launches on
  if (t >= total) {
    // The threads behind the boxes (keys_by_class != null): one per (image, prior) turns the
    // prior's C confidences into sort keys and stores them class by class, [image][class]
    // [prior], so that the launch that orders a class reads its keys front to back.
    const long t2 = t - total;
    if (keys_by_class == nullptr || t2 >= (long)num * P) return;
    const int p = static_cast<int>(t2 % P);
    const int i = static_cast<int>(t2 / P);
    const float* cp = conf + ((long)i * P + p) * C;
    for (int c0 = 0; c0 < C; c0 += 8) {  // eight loads in flight before the first store
      float v[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) v[q] = cp[min(c0 + q, C - 1)];
#pragma unroll
      for (int q = 0; q < 8; ++q)
        if (c0 + q < C) keys_by_class[((long)i * C + c0 + q) * P + p] = desc_key(v[q]);
    }
    return;
  }
  const int p = static_cast<int>(t % P);
  const int c = static_cast<int>((t / P) % loc_classes);
  const int i = static_cast<int>(t / ((long)P * loc_classes));
  const float* l = loc + ((long)i * P + p) * loc_classes * 4 + c * 4;
  const float* pr = prior + p * 4;
  const float* var = prior + ((long)P + p) * 4;
  const float pxmin = pr[0], pymin = pr[1], pxmax = pr[2], pymax = pr[3];
  DBox b;
  if (code_type == 1) {
    if (var_in_target) {
      b.xmin = pxmin + l[0];
      b.ymin = pymin + l[1];
      b.xmax = pxmax + l[2];
      b.ymax = pymax + l[3];
    } else {
      b.xmin = pxmin + var[0] * l[0];
      b.ymin = pymin + var[1] * l[1];
      b.xmax = pxmax + var[2] * l[2];
      b.ymax = pymax + var[3] * l[3];
    }
  } else if (code_type == 2) {
    const float pw = pxmax - pxmin;
    const float ph = pymax - pymin;
    const float pcx = static_cast<float>((static_cast<double>(pxmin + pxmax)) / 2.);
    const float pcy = static_cast<float>((static_cast<double>(pymin + pymax)) / 2.);
    float cx, cy, w, h;
    if (var_in_target) {
      cx = l[0] * pw + pcx;
      cy = l[1] * ph + pcy;
      w = static_cast<float>(exp(static_cast<double>(l[2])) * static_cast<double>(pw));
      h = static_cast<float>(exp(static_cast<double>(l[3])) * static_cast<double>(ph));
    } else {
      cx = var[0] * l[0] * pw + pcx;
      cy = var[1] * l[1] * ph + pcy;
      w = static_cast<float>(exp(static_cast<double>(var[2] * l[2])) * static_cast<double>(pw));
      h = static_cast<float>(exp(static_cast<double>(var[3] * l[3])) * static_cast<double>(ph));
    }
    b.xmin = static_cast<float>(static_cast<double>(cx) - static_cast<double>(w) / 2.);
    b.ymin = static_cast<float>(static_cast<double>(cy) - static_cast<double>(h) / 2.);
    b.xmax = static_cast<float>(static_cast<double>(cx) + static_cast<double>(w) / 2.);
    b.ymax = static_cast<float>(static_cast<double>(cy) + static_cast<double>(h) / 2.);
  } else {
    const float pw = pxmax - pxmin;
    const float ph = pymax - pymin;
    if (var_in_target) {
      b.xmin = pxmin + l[0] * pw;
      b.ymin = pymin + l[1] * ph;
      b.xmax = pxmax + l[2] * pw;
      b.ymax = pymax + l[3] * ph;
    } else {
      b.xmin = pxmin + var[0] * l[0] * pw;
      b.ymin = pymin + var[1] * l[1] * ph;
      b.xmax = pxmax + var[2] * l[2] * pw;
      b.ymax = pymax + var[3] * l[3] * ph;
    }
  }
  b.size = dbox_size(b.xmin, b.ymin, b.xmax, b.ymax);
  out[t] = b;
}

// JaccardOverlap on normalised boxes with cached sizes (bbox_util.cpp:184-204).
__device__ __forceinline__ float jaccard(const DBox& a, const DBox& b) {
  float ixmin, iymin, ixmax, iymax;
  if (b.xmin > a.xmax || b.xmax < a.xmin || b.ymin > a.ymax || b.ymax < a.ymin) {
    ixmin = iymin = ixmax = iymax = 0.f;
  } else {
    ixmin = fmaxf(a.xmin, b.xmin);
    iymin = fmaxf(a.ymin, b.ymin);
    ixmax = fminf(a.xmax, b.xmax);
    iymax = fminf(a.ymax, b.ymax);
  }
  const float iw = ixmax - ixmin, ih = iymax - iymin;
  if (iw > 0.f && ih > 0.f) {
    const float isz = iw * ih;
    return isz / (a.size + b.size - isz);
  }
  return 0.f;
}

// !(JaccardOverlap(a, b) <= thr) in straight-line code: the quotient is formed for
// every pair and used only where the intersection has positive width and height.
// Without the reference's early return for disjoint boxes the intersection's width
// or height comes out negative there (fmaxf / fminf ignore a NaN operand, and the
// comparison that found the boxes disjoint had none), which is overlap 0 as well.
__device__ __forceinline__ bool overlap_rejects(const DBox& a, const DBox& b, float thr) {
  const float iw = fminf(a.xmax, b.xmax) - fmaxf(a.xmin, b.xmin);
  const float ih = fminf(a.ymax, b.ymax) - fmaxf(a.ymin, b.ymin);
  const float isz = iw * ih;
  const float q = isz / (a.size + b.size - isz);
  const float overlap = (iw > 0.f && ih > 0.f) ? q : 0.f;
  return !(overlap <= thr);
}

// The same for the many-pairs kernel, whose second box `b` is the same in every lane (it
// sits in scalar registers).  fmaxf / fminf first quiet a possible signalling NaN in each
// operand the compiler cannot prove clean, one more vector instruction per coordinate of
// `b` and pair; v_max_f32 / v_min_f32 written out take the operands as they are.  For
// ordered operands both give the larger / smaller one; with a NaN coordinate (a NaN location
// prediction) the reference's overlap is not defined either.
__device__ __forceinline__ float vmax_vs(float v, float s) {
  float r;
  asm("v_max_f32 %0, %2, %1" : "=v"(r) : "v"(v), "s"(s));
  return r;
}
__device__ __forceinline__ float vmin_vs(float v, float s) {
  float r;
  asm("v_min_f32 %0, %2, %1" : "=v"(r) : "v"(v), "s"(s));
  return r;
}
__device__ __forceinline__ bool overlap_rejects_uniform_b(const DBox& a, const DBox& b, float thr) {
  const float iw = vmin_vs(a.xmax, b.xmax) - vmax_vs(a.xmin, b.xmin);
  const float ih = vmin_vs(a.ymax, b.ymax) - vmax_vs(a.ymin, b.ymin);
  const float isz = iw * ih;
  const float q = isz / (a.size + b.size - isz);
  const float overlap = (iw > 0.f && ih > 0.f) ? q : 0.f;
  return !(overlap <= thr);
}

constexpr int kKeptLds = 512;  // kept boxes cached in LDS; further ones are read from memory

// The greedy pass of ApplyNMSFast with its adaptive threshold, by one
// wavefront: candidate r is prior cand_idx[r]; its box is cand_box[r] for
// r < n_cached, else read from memory.
template <typename IT>
__device__ __forceinline__ void greedy_nms_wave(int lane, int ncand, int n_cached,
                                                const IT* cand_idx, const DBox* cand_box,
                                                const DBox* cls_boxes, DBox* kept_box, int* kept,
                                                float nms_thr, float eta, int* kept_count_out) {
  float adaptive = nms_thr;
  int nkept = 0;
  for (int r = 0; r < ncand; ++r) {
    const int idx = static_cast<int>(cand_idx[r]);
    const DBox b = r < n_cached ? cand_box[r] : cls_boxes[idx];
    bool reject = false;
    for (int base = 0; base < nkept && !reject; base += 64) {
      const int k = base + lane;
      bool over = false;
      if (k < nkept) {
        const DBox kb = k < kKeptLds ? kept_box[k] : cls_boxes[kept[k]];
        over = !(jaccard(b, kb) <= adaptive);
      }
      reject = __any(over);
    }
    if (!reject) {
      if (lane == 0) {
        kept[nkept] = idx;
        if (nkept < kKeptLds) kept_box[nkept] = b;
      }
      ++nkept;
      if (eta < 1.f && adaptive > 0.5f) adaptive *= eta;
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();
    }
  }
  if (lane == 0) *kept_count_out = nkept;
}

// One workgroup per (image, class).  Candidates: scores above the confidence
// threshold in (score desc, prior index asc) order, cut to top_k; then the
// greedy pass.  This variant sorts through global scratch (any P).
__global__ __launch_bounds__(kSortThreads) void det_class_nms_kernel(
    const float* __restrict__ conf, const DBox* __restrict__ boxes, int P, int C,
    int loc_classes, int background, float conf_thr, float nms_thr, float eta, int top_k,
    int max_cand, uint32_t* keys0, int* vals0, uint32_t* keys1, int* vals1,
    int* __restrict__ kept_idx, int* __restrict__ kept_count) {
  __shared__ BlockSortLds lds;
  __shared__ DBox kept_box[kKeptLds];
  __shared__ int s_valid;
  const int c = blockIdx.x, i = blockIdx.y;
  const int seg = i * C + c;
  if (c == background) {
    if (threadIdx.x == 0) kept_count[seg] = 0;
    return;
  }
  uint32_t* k0 = keys0 + (size_t)seg * P;
  int* v0 = vals0 + (size_t)seg * P;
  uint32_t* k1 = keys1 + (size_t)seg * P;
  int* v1 = vals1 + (size_t)seg * P;
  if (threadIdx.x == 0) s_valid = 0;
  __syncthreads();
  // Contiguous runs per thread, as block_sort_desc expects.
  const int per = (P + kSortThreads - 1) / kSortThreads;
  const int begin = min(static_cast<int>(threadIdx.x) * per, P), end = min(begin + per, P);
  int valid = 0;
  for (int p = begin; p < end; ++p) {
    const float s = conf[((size_t)i * P + p) * C + c];
    const bool ok = s > conf_thr;
    valid += ok;
    k0[p] = ok ? desc_key(s) : 0xffffffffu;  // below-threshold scores sort last
    v0[p] = p;
  }
  if (valid) atomicAdd(&s_valid, valid);
  __syncthreads();
  block_sort_desc(k0, v0, k1, v1, P, &lds);
  int ncand = s_valid;
  if (top_k > -1 && top_k < ncand) ncand = top_k;
  const DBox* cls_boxes = boxes + ((size_t)i * loc_classes + (loc_classes == 1 ? 0 : c)) * P;
  // The serial greedy pass would pay one dependent global load pair per
  // candidate: the whole workgroup fetches the first candidates' indices and
  // boxes into the (now free) histogram storage first.
  constexpr int kCandLds = static_cast<int>(sizeof(lds.counts) / (sizeof(DBox) + sizeof(int)));
  DBox* cand_box = reinterpret_cast<DBox*>(lds.counts);
  int* cand_idx = reinterpret_cast<int*>(cand_box + kCandLds);
  __syncthreads();
  for (int r = threadIdx.x; r < min(ncand, kCandLds); r += kSortThreads) {
    const int idx = v0[r];
    cand_idx[r] = idx;
    cand_box[r] = cls_boxes[idx];
  }
  __syncthreads();
  if (threadIdx.x >= 64) return;  // the greedy pass is one wavefront
  // with more candidates than the cache holds, indices come from the sorted list in memory
  greedy_nms_wave<int>(threadIdx.x, ncand, min(ncand, kCandLds), ncand <= kCandLds ? cand_idx : v0,
                       cand_box, cls_boxes, kept_box, kept_idx + (size_t)seg * max_cand, nms_thr,
                       eta, &kept_count[seg]);
}

// The greedy pass for a constant threshold (eta == 1), 64 candidates (a block) at a
// time, by the whole workgroup.  "Candidate r is rejected against a kept k < r" does
// not depend on the order of decisions when the threshold is fixed, so the tests
// can run in parallel: a wavefront holds candidate 64 w + l in lane l, tests it
// against a candidate k (a broadcast read) and a ballot is word w of k's row.
//   1. the block's own pairs (all wavefronts, eight of the block's candidates each as
//      the earlier box): lane l collects in `before[l]` the earlier candidates of the block
//      that candidate l is rejected against;
//   2. one wavefront decides the block in rounds: a candidate none of whose rejecting
//      predecessors is still open is settled, rejected if one of them is kept, else kept
//      (two ballots per round; the first open candidate always settles, and candidates
//      reject few of their neighbours, so a few rounds instead of one step per kept
//      candidate); the kept ones are written by their lanes;
//   3. only the rows of the candidates kept in this block are evaluated against the
//      later blocks (all wavefronts) and OR-ed into the rejected set, one word per
//      later block.  Rows of rejected candidates are never formed.
// State: `later[w]` = word w of the rejected set, `before[l]`, one word of kept bits.
constexpr int kDetCandBoxes = 1024;  // candidates whose boxes are cached in LDS
struct BlockNmsLds {
  unsigned long long later[kDetCandBoxes / 64];
  unsigned long long before[64];  // per candidate of the block: the earlier ones of the block it is rejected against
  unsigned long long keep;
  int kept_list[64];
};
template <typename IT>
__device__ __forceinline__ void greedy_nms_blocks(int ncand, const IT* cand_idx,
                                                  const DBox* cand_box, BlockNmsLds* st,
                                                  int* kept, float nms_thr, int* kept_count_out) {
  const int words = (ncand + 63) >> 6;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr int kWaves = kSortThreads / 64;
  if (threadIdx.x < kDetCandBoxes / 64) st->later[threadIdx.x] = 0;
  if (threadIdx.x < 64) st->before[threadIdx.x] = 0;
  int nkept = 0;  // used by wavefront 0
  __syncthreads();
  for (int blk = 0; blk < words; ++blk) {
    const int bn = min(64, ncand - 64 * blk);
    {
      // 1. the block's own pairs: lane l collects the earlier candidates of the block that
      // candidate 64 blk + l is rejected against (the test is symmetric in its two boxes)
      const int r = 64 * blk + lane;
      const bool in = r < ncand;
      const DBox rb = cand_box[min(r, ncand - 1)];
      constexpr int kPer = 64 / kWaves;
      unsigned long long mine = 0;
#pragma unroll 1
      for (int i0 = wave * kPer; i0 < min(wave * kPer + kPer, bn); i0 += 4) {
        DBox kb[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) kb[q] = cand_box[64 * blk + min(i0 + q, bn - 1)];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const bool hit = in & (lane > i0 + q) & (i0 + q < bn) & overlap_rejects(rb, kb[q], nms_thr);
          mine |= hit ? 1ull << (i0 + q) : 0ull;
        }
      }
      if (mine) atomicOr(&st->before[lane], mine);
    }
    __syncthreads();
    if (wave == 0) {
      // 2. decide the block in rounds: a candidate none of whose rejecting predecessors is
      // still open is settled, rejected if one of them is kept, else kept.  The first open
      // candidate always settles; candidates reject few of their neighbours, so a few rounds.
      const unsigned long long before = st->before[lane];
      st->before[lane] = 0;  // for the next block (two barriers away)
      const unsigned long long valid = bn >= 64 ? ~0ull : ((1ull << bn) - 1ull);
      const unsigned long long prior = st->later[blk];
      // (readfirstlane returns a signed int: through unsigned, or the low half would sign-extend)
      const unsigned b_lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(prior));
      const unsigned b_hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(prior >> 32));
      const unsigned long long rem = (static_cast<unsigned long long>(b_hi) << 32) | b_lo;
      unsigned long long open = ~rem & valid, keep_bits = 0;
      while (open != 0) {  // wave-uniform
        const bool is_open = (open >> lane) & 1ull;
        const bool rejected = (before & keep_bits) != 0;
        const bool waits = (before & open) != 0;
        const unsigned long long now_rejected = __ballot(is_open && rejected);
        const unsigned long long now_kept = __ballot(is_open && !rejected && !waits);
        keep_bits |= now_kept;
        open &= ~(now_kept | now_rejected);
      }
      // the block's kept candidates, in order, by their own lanes
      if ((keep_bits >> lane) & 1ull) {
        const int pos = __popcll(keep_bits & ((1ull << lane) - 1ull));
        kept[nkept + pos] = static_cast<int>(cand_idx[64 * blk + lane]);
        st->kept_list[pos] = 64 * blk + lane;
      }
      nkept += __popcll(keep_bits);
      if (lane == 0) st->keep = keep_bits;
    }
    if (blk + 1 == words) break;  // uniform over the workgroup
    __syncthreads();
    {
      // 3. kept rows against the later blocks.  nw later words for kWaves wavefronts:
      // with fewer words than wavefronts each word's kept rows are shared by several.
      const int nk = __popcll(st->keep);
      const int nw = words - blk - 1;
      const int groups = nw >= kWaves ? 1 : kWaves / nw;  // wavefronts per word
      for (int item = wave; item < nw * groups; item += kWaves) {
        const int w = blk + 1 + item % nw, g = item / nw;
        const int r = 64 * w + lane;
        const bool in = r < ncand;
        const DBox rb = cand_box[min(r, ncand - 1)];
        unsigned long long acc = 0;
#pragma unroll 1
        for (int t0 = g; t0 < nk; t0 += 4 * groups) {
          DBox kb[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) kb[q] = cand_box[st->kept_list[min(t0 + q * groups, nk - 1)]];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            // (no short-circuit: four straight-line overlaps the scheduler can interleave)
            const unsigned long long bits = __ballot(
                static_cast<int>(in) & static_cast<int>(overlap_rejects(rb, kb[q], nms_thr)));
            if (t0 + q * groups < nk) acc |= bits;
          }
        }
        if (lane == 0 && acc) atomicOr(&st->later[w], acc);
      }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) *kept_count_out = nkept;
}

// The same for P <= kDetLdsMax priors: scores are keyed straight into LDS and
// sorted there (no global scratch traffic), the sorted prior indices double as
// the candidate list.
constexpr int kDetLdsPer = 24;
constexpr int kDetLdsMax = kDetLdsPer * kSortThreads;  // 12288
__global__ __launch_bounds__(kSortThreads) void det_class_nms_lds_kernel(
    const float* __restrict__ conf, const DBox* __restrict__ boxes, int P, int C,
    int loc_classes, int background, float conf_thr, float nms_thr, float eta, int top_k,
    int max_cand, int* __restrict__ kept_idx, int* __restrict__ kept_count) {
  __shared__ BlockSortLds16 lds;
  __shared__ __attribute__((aligned(8))) uint32_t s_key[kDetLdsMax];
  __shared__ unsigned short s_val[kDetLdsMax];
  __shared__ DBox cand_box[kDetCandBoxes];
  __shared__ DBox kept_box[kKeptLds];
  __shared__ int s_valid;
  const int c = blockIdx.x, i = blockIdx.y;
  const int seg = i * C + c;
  if (c == background) {
    if (threadIdx.x == 0) kept_count[seg] = 0;
    return;
  }
  if (threadIdx.x == 0) s_valid = 0;
  __syncthreads();
  int valid = 0;
  // eight independent loads in flight per thread: the launch is one workgroup per CU
  constexpr int kLoads = 8;
  for (int p0 = threadIdx.x; p0 < P; p0 += kSortThreads * kLoads) {
    float sc[kLoads];
#pragma unroll
    for (int q = 0; q < kLoads; ++q) {
      const int p = p0 + q * kSortThreads;
      sc[q] = p < P ? conf[((size_t)i * P + p) * C + c] : 0.f;
    }
#pragma unroll
    for (int q = 0; q < kLoads; ++q) {
      const int p = p0 + q * kSortThreads;
      if (p < P) {
        const bool ok = sc[q] > conf_thr;
        valid += ok;
        s_key[p] = ok ? desc_key(sc[q]) : 0xffffffffu;  // below-threshold scores sort last
        s_val[p] = static_cast<unsigned short>(p);
      }
    }
  }
  if (valid) atomicAdd(&s_valid, valid);
  __syncthreads();
  // Only scores above the threshold can become candidates: squeeze them to the
  // front in prior order (a stable sort of the survivors alone gives the order the
  // sort of all priors would give them) and sort just those.
  const int nvalid = s_valid;
  if (nvalid < P) {
    const int per = (P + kSortThreads - 1) / kSortThreads;
    const int begin = min(static_cast<int>(threadIdx.x) * per, P), end = min(begin + per, P);
    uint32_t rk[kDetLdsPer];
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < kDetLdsPer; ++j) {
      rk[j] = 0xffffffffu;
      if (begin + j < end) rk[j] = s_key[begin + j];
      mine += rk[j] != 0xffffffffu;
    }
    uint32_t pos = block_exclusive_scan(mine, lds.wave_sum);  // synchronises before returning
#pragma unroll
    for (int j = 0; j < kDetLdsPer; ++j)
      if (rk[j] != 0xffffffffu) {
        s_key[pos] = rk[j];
        s_val[pos] = static_cast<unsigned short>(begin + j);
        ++pos;
      }
    __syncthreads();
  }
  block_sort_desc_lds<kDetLdsPer, unsigned short>(s_key, s_val, nvalid, &lds);
  int ncand = nvalid;
  if (top_k > -1 && top_k < ncand) ncand = top_k;
  const DBox* cls_boxes = boxes + ((size_t)i * loc_classes + (loc_classes == 1 ? 0 : c)) * P;
  const int n_cached = min(ncand, kDetCandBoxes);
  for (int r = threadIdx.x; r < n_cached; r += kSortThreads) cand_box[r] = cls_boxes[s_val[r]];
  __syncthreads();
  // constant threshold: the workgroup's block-wise pass; otherwise the greedy pass of
  // one wavefront
  if (eta >= 1.f && ncand <= kDetCandBoxes) {
    greedy_nms_blocks<unsigned short>(ncand, s_val, cand_box,
                                      reinterpret_cast<BlockNmsLds*>(s_key),
                                      kept_idx + (size_t)seg * max_cand, nms_thr, &kept_count[seg]);
    return;
  }
  if (threadIdx.x >= 64) return;  // the greedy pass is one wavefront
  greedy_nms_wave<unsigned short>(threadIdx.x, ncand, n_cached, s_val, cand_box, cls_boxes, kept_box,
                                  kept_idx + (size_t)seg * max_cand, nms_thr, eta,
                                  &kept_count[seg]);
}

// ---- constant threshold, top_k <= 512, P <= kDetLdsMax: the per-class work in three launches
//
// det_candidates_kernel (one workgroup per image and class) picks and orders the class's
// top_k candidates; det_overlap_kernel forms the candidates' pairwise "rejects" bits with
// one wavefront per 64 x 64 block of pairs, so the quadratic part of the work spreads
// over the whole chip instead of one CU per class; det_scan_kernel (one wavefront per
// image and class) makes the greedy decisions from those bits alone.
constexpr int kDetSplitTopK = kSortThreads;          // candidates per class at most
constexpr int kDetSplitWords = kDetSplitTopK / 64;   // 64-candidate blocks per class at most

// The candidates by a sort of the whole key table in LDS, for tables the selection gives up
// on.  Kept out of line: inlined, its register arrays spill the selection's.
__device__ __noinline__ int det_candidates_by_sort(const uint32_t* __restrict__ keys, int P, uint32_t key_thr,
                                                   int want, uint32_t* s_key, unsigned short* s_val,
                                                   BlockSortLds16* lds, int* s_valid, uint32_t* key_out,
                                                   uint32_t* idx_out) {
  const int tid = threadIdx.x;
  if (tid == 0) *s_valid = 0;
  __syncthreads();
  int valid = 0;
  for (int p = tid; p < P; p += kSortThreads) {
    const uint32_t k = keys[p];
    const bool ok = k < key_thr;
    valid += ok;
    s_key[p] = ok ? k : 0xffffffffu;  // below-threshold scores sort last
    s_val[p] = static_cast<unsigned short>(p);
  }
  if (valid) atomicAdd(s_valid, valid);
  __syncthreads();
  // squeeze the scores above the threshold to the front in prior order and sort those
  const int nvalid = *s_valid;
  if (nvalid < P) {
    const int per = (P + kSortThreads - 1) / kSortThreads;
    const int begin = min(tid * per, P), end = min(begin + per, P);
    uint32_t run[kDetLdsPer];
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < kDetLdsPer; ++j) {
      run[j] = 0xffffffffu;
      if (begin + j < end) run[j] = s_key[begin + j];
      mine += run[j] != 0xffffffffu;
    }
    uint32_t pos = block_exclusive_scan(mine, lds->wave_sum);  // synchronises before returning
#pragma unroll
    for (int j = 0; j < kDetLdsPer; ++j)
      if (run[j] != 0xffffffffu) {
        s_key[pos] = run[j];
        s_val[pos] = static_cast<unsigned short>(begin + j);
        ++pos;
      }
    __syncthreads();
  }
  block_sort_desc_lds<kDetLdsPer, unsigned short>(s_key, s_val, nvalid, lds);
  const int ncand = min(nvalid, want);
  if (tid < ncand) {
    *key_out = s_key[tid];
    *idx_out = s_val[tid];
  }
  return ncand;
}

// Candidates of one (image, class): the top_k best scores above the threshold in (score
// descending, prior ascending) order, what GetMaxScoreIndex leaves (bbox_util.cpp:523-540).
// The keys come class by class from det_decode_kernel; a score is above the threshold
// exactly if its key is below the threshold's key.  First the selection that does not sort
// the table; if it gives up (crowds of equal scores), the sort in LDS.
__global__ __launch_bounds__(kSortThreads) void det_candidates_kernel(
    const uint32_t* __restrict__ keys_by_class, const DBox* __restrict__ boxes, int P, int C,
    int loc_classes, int background, uint32_t key_thr, int top_k, int cand_stride,
    uint32_t* __restrict__ cand_key, int* __restrict__ cand_idx, DBox* __restrict__ cand_box,
    int* __restrict__ ncand_out) {
  __shared__ BlockSortLds16 lds;
  __shared__ __attribute__((aligned(16))) uint32_t s_key[kDetLdsMax];
  __shared__ unsigned short s_val[kDetLdsMax];
  __shared__ int s_valid;
  static_assert(sizeof(BlockSelectLds) <= sizeof(uint32_t) * kDetLdsMax, "the selection's scratch overlays the key table");
  const int c = blockIdx.x, i = blockIdx.y;
  const int seg = i * C + c;
  const int tid = threadIdx.x;
  if (c == background) {
    if (tid == 0) ncand_out[seg] = 0;
    return;
  }
  const uint32_t* __restrict__ keys = keys_by_class + (size_t)seg * P;
  uint32_t rk[kDetLdsPer];
#pragma unroll
  for (int j = 0; j < kDetLdsPer; ++j) {
    const int p = tid + j * kSortThreads;
    rk[j] = p < P ? keys[p] : 0xffffffffu;
  }
  const int want = min(top_k, P);
  uint32_t key = 0xffffffffu, idx = 0;
  int ncand;
  const int m = block_select_smallest<kDetLdsPer>(rk, want, reinterpret_cast<BlockSelectLds*>(s_key), &key, &idx);
  if (m > 0) {  // uniform
    ncand = __syncthreads_count(tid < want && key < key_thr);
  } else {
    // (its results through variables of their own: a variable whose address goes to a
    // function that is not inlined lives in scratch memory for the whole kernel)
    uint32_t sorted_key = 0xffffffffu, sorted_idx = 0;
    ncand = det_candidates_by_sort(keys, P, key_thr, want, s_key, s_val, &lds, &s_valid, &sorted_key,
                                   &sorted_idx);
    key = sorted_key;
    idx = sorted_idx;
  }
  if (tid < ncand) {
    const DBox* cls_boxes = boxes + ((size_t)i * loc_classes + (loc_classes == 1 ? 0 : c)) * P;
    const size_t at = (size_t)seg * cand_stride + tid;
    cand_key[at] = key;
    cand_idx[at] = static_cast<int>(idx);
    cand_box[at] = cls_boxes[idx];
  }
  if (tid == 0) ncand_out[seg] = ncand;
}

// One wavefront per pair of 64-candidate blocks (bi <= bj) of one (image, class): lane l
// holds candidate 64 bi + l (the earlier box of a pair) and candidate 64 bj + l; the later
// boxes go round as scalar broadcasts, and a ballot over the earlier ones is the word the
// scan needs: col_rejects[candidate 64 bj + k][bi] = the candidates of block bi that
// candidate 64 bj + k is rejected against (JaccardOverlap is symmetric in its two boxes:
// bbox_util.cpp:184-204).
constexpr int kOverlapWaves = 4;
__global__ __launch_bounds__(64 * kOverlapWaves) void det_overlap_kernel(
    const DBox* __restrict__ cand_box, const int* __restrict__ ncand_in, int cand_stride, float nms_thr,
    unsigned long long* __restrict__ col_rejects) {
  const int seg = blockIdx.y;
  const int lane = threadIdx.x & 63;
  // pair index bj (bj + 1) / 2 + bi (the same in every lane: said so, for scalar addressing)
  const int q = blockIdx.x * kOverlapWaves + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int bj = 0;
  while ((bj + 1) * (bj + 2) / 2 <= q) ++bj;
  const int bi = q - bj * (bj + 1) / 2;
  const int ncand = ncand_in[seg];
  if (64 * bj >= ncand) return;  // (uniform over the wavefront; bi <= bj)
  const DBox* __restrict__ cb = cand_box + (size_t)seg * cand_stride;
  const int r = 64 * bi + lane, k0 = 64 * bj + lane;
  const bool row_in = r < ncand;
  const DBox rb = cb[min(r, ncand - 1)];
  // The later box of a pair is the same for the whole wavefront: read through the scalar
  // unit (a uniform address in memory nobody writes during the launch), so the vector unit
  // only does the arithmetic.  Columns past the last candidate repeat it; their words are
  // never read.
  unsigned long long word = 0;
#pragma unroll 8
  for (int k = 0; k < 64; ++k) {
    const DBox kb = cb[min(64 * bj + k, ncand - 1)];
    const unsigned long long bits =
        __ballot(static_cast<int>(row_in) & static_cast<int>(overlap_rejects_uniform_b(rb, kb, nms_thr)));
    word = lane == k ? bits : word;
  }
  col_rejects[((size_t)seg * cand_stride + k0) * kDetSplitWords + bi] = word;  // (k0 < 64 words <= cand_stride)
}

// The greedy pass of ApplyNMSFast for a constant threshold (bbox_util.cpp:681-716) from the
// bits alone, one wavefront per (image, class), a block of 64 candidates at a time: a
// candidate is out if a kept candidate of an earlier block rejects it (its words of the
// earlier blocks against those blocks' kept bits); the block's own candidates settle in
// rounds as in greedy_nms_blocks.  Every word a lane will need is requested before the
// first decision, so the pass waits for memory once.
__global__ __launch_bounds__(64) void det_scan_kernel(
    const unsigned long long* __restrict__ col_rejects, const int* __restrict__ ncand_in,
    const int* __restrict__ cand_idx, const uint32_t* __restrict__ cand_key,
    const DBox* __restrict__ cand_box, int cand_stride, int max_cand, int* __restrict__ kept_idx,
    uint32_t* __restrict__ kept_key, DBox* __restrict__ kept_box, int* __restrict__ kept_count) {
  const int seg = blockIdx.x, lane = threadIdx.x;
  const int ncand = ncand_in[seg];
  const int words = (ncand + 63) >> 6;
  unsigned long long w[kDetSplitWords][kDetSplitWords];
  int prior[kDetSplitWords];
  uint32_t ckey[kDetSplitWords];
  float cbox[kDetSplitWords][5];  // (five floats each: an array of DBox would live in scratch memory)
  static_assert(sizeof(DBox) == 5 * sizeof(float), "a box is five floats");
#pragma unroll
  for (int b = 0; b < kDetSplitWords; ++b) {
    if (b < words) {  // uniform
      const size_t at = (size_t)seg * cand_stride + 64 * b + lane;
      const ulonglong2* src = reinterpret_cast<const ulonglong2*>(col_rejects + at * kDetSplitWords);
#pragma unroll
      for (int h = 0; h < kDetSplitWords / 2; ++h) {
        const ulonglong2 v = src[h];
        w[b][2 * h] = v.x;
        w[b][2 * h + 1] = v.y;
      }
      const size_t mine = (size_t)seg * cand_stride + min(64 * b + lane, ncand - 1);
      prior[b] = cand_idx[mine];
      ckey[b] = cand_key[mine];
      const float* box = reinterpret_cast<const float*>(cand_box + mine);
#pragma unroll
      for (int k = 0; k < 5; ++k) cbox[b][k] = box[k];
    }
  }
  unsigned long long keep[kDetSplitWords];
  int nkept = 0;
  int* const kept = kept_idx + (size_t)seg * max_cand;
#pragma unroll
  for (int b = 0; b < kDetSplitWords; ++b) {
    if (b < words) {  // uniform
      const int bn = min(64, ncand - 64 * b);
      const unsigned long long valid = bn >= 64 ? ~0ull : ((1ull << bn) - 1ull);
      bool out = false;
#pragma unroll
      for (int e = 0; e < b; ++e) out = out || (w[b][e] & keep[e]) != 0;
      const unsigned long long before = w[b][b] & ((1ull << lane) - 1ull);
      unsigned long long open = ~__ballot(out) & valid, keep_bits = 0;
      while (open != 0) {  // wave-uniform
        const bool is_open = (open >> lane) & 1ull;
        const bool rejected = (before & keep_bits) != 0;
        const bool waits = (before & open) != 0;
        const unsigned long long now_rejected = __ballot(is_open && rejected);
        const unsigned long long now_kept = __ballot(is_open && !rejected && !waits);
        keep_bits |= now_kept;
        open &= ~(now_kept | now_rejected);
      }
      keep[b] = keep_bits;
      if ((keep_bits >> lane) & 1ull) {
        const int pos = nkept + __popcll(keep_bits & ((1ull << lane) - 1ull));
        kept[pos] = prior[b];
        kept_key[(size_t)seg * max_cand + pos] = ckey[b];
        float* box = reinterpret_cast<float*>(kept_box + (size_t)seg * max_cand + pos);
#pragma unroll
        for (int k = 0; k < 5; ++k) box[k] = cbox[b][k];
      }
      nkept += __popcll(keep_bits);
    }
  }
  if (lane == 0) kept_count[seg] = nkept;
}

// Sum of one int per thread over the workgroup, returned to every thread.  `slots` has
// one entry per wavefront and may be reused right after the call returns.
__device__ __forceinline__ int block_sum(int v, uint32_t* slots) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  if ((threadIdx.x & 63) == 0) slots[threadIdx.x >> 6] = static_cast<uint32_t>(v);
  __syncthreads();
  int total = 0;
#pragma unroll
  for (int w = 0; w < kSortThreads / 64; ++w) total += static_cast<int>(slots[w]);
  __syncthreads();
  return total;
}

constexpr int kSelLdsPer = 16;
constexpr int kSelLdsMax = kSelLdsPer * kSortThreads;  // 8192 entries held in registers (SSD300: 20 classes x 400)

// keep_top_k and the rows of one image whose entry list has at most kSelLdsMax entries:
// every thread keeps its run of up to kSelLdsPer entries (class, prior, score) in
// registers from the first gather to the rows, so the list is read once.
struct SelectShortLds {
  uint32_t slots[2][kSortThreads / 64];
  uint32_t scan[kSortThreads / 64];
  // first entry of every thread's run, for the neighbour test across two runs
  int first_cls[kSortThreads];
  float first_score[kSortThreads];
  unsigned char first_in[kSortThreads];
};
__device__ __forceinline__ void select_short(
    const float* __restrict__ conf, const DBox* __restrict__ boxes, int P, int C, int loc_classes,
    int keep_top_k, int max_cand, const int* __restrict__ kept_idx, const int* s_off, int total,
    int i, float* __restrict__ rows_image, int* __restrict__ rows_count,
    int* __restrict__ cut_tie_flag, SelectShortLds* st) {
  const int tid = threadIdx.x;
  const int per = (total + kSortThreads - 1) / kSortThreads;
  const int begin = min(tid * per, total), end = min(begin + per, total);
  const int cnt = end - begin;
  // first all prior indices, then all scores: two rounds of loads per thread
  int cls[kSelLdsPer], idx[kSelLdsPer];
  float sc[kSelLdsPer];
  {
    int c = 0;
#pragma unroll
    for (int q = 0; q < kSelLdsPer; ++q) {
      cls[q] = 0;
      idx[q] = 0;
      if (q < cnt) {
        const int e = begin + q;
        while (s_off[c + 1] <= e) ++c;
        cls[q] = c;
        idx[q] = kept_idx[(size_t)(i * C + c) * max_cand + (e - s_off[c])];
      }
    }
#pragma unroll
    for (int q = 0; q < kSelLdsPer; ++q)
      sc[q] = q < cnt ? conf[((size_t)i * P + idx[q]) * C + cls[q]] : 0.f;
  }
  uint32_t in_mask = cnt >= 32 ? 0xffffffffu : ((1u << cnt) - 1u);  // bit q: entry begin + q is kept
  if (keep_top_k > -1 && total > keep_top_k) {
    // Which entries are among the keep_top_k best needs no sort: T = the keep_top_k-th
    // smallest key, found bit by bit from the top with one count over the workgroup per
    // bit; entries with a smaller key are in, those equal to T fill the remaining places
    // in entry order -- what a stable sort cut at keep_top_k selects.  The counts: ballots
    // within a wavefront (scalar population counts), the eight wavefront counts through
    // LDS with one barrier (two alternating sets of slots: a set is rewritten two rounds
    // later, when every reader has passed the barrier in between).  Unused register slots
    // hold the largest key; `padding` takes them out of a count that reaches it.
    uint32_t rk[kSelLdsPer];
#pragma unroll
    for (int q = 0; q < kSelLdsPer; ++q) rk[q] = q < cnt ? desc_key(sc[q]) : 0xffffffffu;
    const int padding = kSortThreads * kSelLdsPer - total;
    uint32_t T = 0;
    int parity = 0;
    for (int bit = 31; bit >= 0 && keep_top_k > 0; --bit) {
      const uint32_t mid = T | ((1u << bit) - 1u);
      int below = 0;  // of this wavefront
#pragma unroll
      for (int q = 0; q < kSelLdsPer; ++q) below += __popcll(__ballot(rk[q] <= mid));
      if ((tid & 63) == 0) st->slots[parity][tid >> 6] = static_cast<uint32_t>(below);
      __syncthreads();
      const uint4 a = *reinterpret_cast<const uint4*>(&st->slots[parity][0]);
      const uint4 b = *reinterpret_cast<const uint4*>(&st->slots[parity][4]);
      static_assert(kSortThreads / 64 == 8, "eight wavefront counts");
      int total_below = static_cast<int>(a.x + a.y + a.z + a.w + b.x + b.y + b.z + b.w);
      if (mid == 0xffffffffu) total_below -= padding;
      if (total_below < keep_top_k) T |= 1u << bit;
      parity ^= 1;
    }
    int less = 0, equal = 0;
#pragma unroll
    for (int q = 0; q < kSelLdsPer; ++q) {
      less += (q < cnt) && rk[q] < T;
      equal += (q < cnt) && rk[q] == T;
    }
    const int need_equal = keep_top_k - block_sum(less, st->scan);
    const int equal_total = block_sum(equal, st->scan);
    int rank = static_cast<int>(block_exclusive_scan(static_cast<uint32_t>(equal), st->scan));
    in_mask = 0;
#pragma unroll
    for (int q = 0; q < kSelLdsPer; ++q)
      if (q < cnt) {
        bool in = rk[q] < T;
        if (rk[q] == T) in = rank++ < need_equal;
        in_mask |= static_cast<uint32_t>(in) << q;
      }
    // Equal scores on both sides of the cut: which of them survive is decided here
    // by (label, NMS order) and in the reference by std::sort's internals.
    if (tid == 0 && cut_tie_flag && keep_top_k > 0 && equal_total > need_equal)
      atomicOr(cut_tie_flag, 1);
    // Equal scores of one label among the kept entries: the reference rebuilds each
    // label's list in std::sort's order, here they stay in NMS order.
    if (cut_tie_flag) {
      st->first_cls[tid] = cnt > 0 ? cls[0] : -1;
      st->first_score[tid] = sc[0];
      st->first_in[tid] = static_cast<unsigned char>(in_mask & 1u);
      __syncthreads();
      bool tied = false;
#pragma unroll
      for (int q = 0; q < kSelLdsPer; ++q) {
        if (q >= cnt || !((in_mask >> q) & 1u)) continue;
        if (q + 1 < cnt) {
          tied = tied || (((in_mask >> (q + 1)) & 1u) && cls[q + 1] == cls[q] && sc[q + 1] == sc[q]);
        } else if (tid + 1 < kSortThreads && begin + q + 1 < total) {
          // the next entry opens the next thread's run (runs are contiguous and in order)
          tied = tied || (st->first_in[tid + 1] && st->first_cls[tid + 1] == cls[q] &&
                          st->first_score[tid + 1] == sc[q]);
        }
      }
      if (tied) atomicOr(cut_tie_flag, 2);
    }
  }
  // the kept entries in entry order
  uint32_t pos = block_exclusive_scan(static_cast<uint32_t>(__popc(in_mask)), st->scan);
  DBox bx[kSelLdsPer];
#pragma unroll
  for (int q = 0; q < kSelLdsPer; ++q)
    if ((in_mask >> q) & 1u)
      bx[q] = boxes[((size_t)i * loc_classes + (loc_classes == 1 ? 0 : cls[q])) * P + idx[q]];
#pragma unroll
  for (int q = 0; q < kSelLdsPer; ++q)
    if ((in_mask >> q) & 1u) {
      float* row = rows_image + static_cast<size_t>(pos) * 7;
      row[0] = static_cast<float>(i);
      row[1] = static_cast<float>(cls[q]);
      row[2] = sc[q];
      row[3] = bx[q].xmin;
      row[4] = bx[q].ymin;
      row[5] = bx[q].xmax;
      row[6] = bx[q].ymax;
      ++pos;
    }
  if (tid == kSortThreads - 1) rows_count[i] = static_cast<int>(pos);
}

// One workgroup per image: applies keep_top_k over all classes and writes the
// image's rows [image, label, score, xmin, ymin, xmax, ymax], labels ascending,
// each label's boxes in NMS order.
__global__ __launch_bounds__(kSortThreads) void det_select_kernel(
    const float* __restrict__ conf, const DBox* __restrict__ boxes, int P, int C,
    int loc_classes, int keep_top_k, int max_cand, const int* __restrict__ kept_idx,
    const int* __restrict__ kept_count, uint32_t* keys0, int* vals0, uint32_t* keys1,
    int* vals1, int* __restrict__ selected, float* __restrict__ rows_tmp,
    int* __restrict__ rows_count, int* __restrict__ cut_tie_flag) {
  __shared__ BlockSortLds lds;
  __shared__ SelectShortLds short_lds;
  __shared__ int s_off[1024];  // start of each class in the image's entry list
  const int i = blockIdx.x;
  const int max_entries = C * max_cand;
  uint32_t* k0 = keys0 + (size_t)i * max_entries;
  int* v0 = vals0 + (size_t)i * max_entries;
  uint32_t* k1 = keys1 + (size_t)i * max_entries;
  int* v1 = vals1 + (size_t)i * max_entries;
  int* sel = selected + (size_t)i * max_entries;
  // (the counts are fetched by one thread each: a single thread adding them up straight
  // from memory would pay one load latency per class)
  for (int c = threadIdx.x; c < C; c += kSortThreads) s_off[c + 1] = kept_count[i * C + c];
  __syncthreads();
  if (threadIdx.x == 0) {
    int off = 0;
    for (int c = 0; c < C; ++c) {
      const int cnt = s_off[c + 1];
      s_off[c] = off;
      off += cnt;
    }
    s_off[C] = off;
  }
  __syncthreads();
  const int total = s_off[C];
  // entry e = (label, position in that label's NMS order), labels ascending
  if (total <= kSelLdsMax) {  // uniform
    select_short(conf, boxes, P, C, loc_classes, keep_top_k, max_cand, kept_idx, s_off, total, i,
                 rows_tmp + (size_t)i * max_entries * 7, rows_count, cut_tie_flag, &short_lds);
    return;
  }
  // Longer lists go through global scratch: flags, a stable sort cut at keep_top_k.
  for (int e = threadIdx.x; e < total; e += kSortThreads) sel[e] = 1;
  __syncthreads();
  const int per = (total + kSortThreads - 1) / kSortThreads;
  const int begin = min(static_cast<int>(threadIdx.x) * per, total), end = min(begin + per, total);
  if (keep_top_k > -1 && total > keep_top_k) {
    {
      int c = 0;
      for (int e = begin; e < end; ++e) {
        while (s_off[c + 1] <= e) ++c;
        const int idx = kept_idx[(size_t)(i * C + c) * max_cand + (e - s_off[c])];
        k0[e] = desc_key(conf[((size_t)i * P + idx) * C + c]);
        v0[e] = e;
      }
    }
    __syncthreads();
    block_sort_desc(k0, v0, k1, v1, total, &lds);
    for (int r = threadIdx.x; r < total; r += kSortThreads) sel[v0[r]] = r < keep_top_k;
    // Equal scores on both sides of the cut: which of them survive is decided here
    // by (label, NMS order) and in the reference by std::sort's internals.
    if (threadIdx.x == 0 && cut_tie_flag && keep_top_k > 0 && k0[keep_top_k - 1] == k0[keep_top_k])
      atomicOr(cut_tie_flag, 1);
    __syncthreads();
    // Equal scores of one label among the kept entries: the reference rebuilds each
    // label's list in std::sort's order, here they stay in NMS order.
    if (cut_tie_flag) {
      int cc = 0;
      bool tied = false;
      for (int e = begin; e < end; ++e) {
        while (s_off[cc + 1] <= e) ++cc;
        if (!sel[e] || e + 1 >= s_off[cc + 1] || !sel[e + 1]) continue;
        const int* list = kept_idx + (size_t)(i * C + cc) * max_cand;
        const float a = conf[((size_t)i * P + list[e - s_off[cc]]) * C + cc];
        const float b = conf[((size_t)i * P + list[e + 1 - s_off[cc]]) * C + cc];
        tied = tied || a == b;
      }
      if (tied) atomicOr(cut_tie_flag, 2);
    }
    __syncthreads();
  }
  // compact the selected entries in entry order (a block scan over `sel`)
  uint32_t mine = 0;
  for (int e = begin; e < end; ++e) mine += sel[e];
  uint32_t pos = block_exclusive_scan(mine, lds.wave_sum);
  int c = 0;
  for (int e = begin; e < end; ++e) {
    if (!sel[e]) continue;
    while (s_off[c + 1] <= e) ++c;
    const int idx = kept_idx[(size_t)(i * C + c) * max_cand + (e - s_off[c])];
    const DBox b = boxes[((size_t)i * loc_classes + (loc_classes == 1 ? 0 : c)) * P + idx];
    float* row = rows_tmp + ((size_t)i * max_entries + pos) * 7;
    row[0] = static_cast<float>(i);
    row[1] = static_cast<float>(c);
    row[2] = conf[((size_t)i * P + idx) * C + c];
    row[3] = b.xmin;
    row[4] = b.ymin;
    row[5] = b.xmax;
    row[6] = b.ymax;
    ++pos;
  }
  __syncthreads();
  if (threadIdx.x == kSortThreads - 1) rows_count[i] = static_cast<int>(pos);
}

// keep_top_k and the output rows of one image from what det_scan_kernel left (keys and
// boxes of every class's kept candidates in NMS order), for keep_top_k <= 512 and at most
// kSelLdsMax entries per image; the rows go straight to their place in the output (every
// workgroup adds up the row counts of the images before its own), so no launch follows.
// The keep_top_k best entries come from the selection that does not sort the list; ties
// at the cut go by (label, NMS order), which is entry order.  If the selection gives up,
// select_short does the image the long way round.
struct SelectFastLds {
  BlockSelectLds sel;
  int rows[1024];  // rows of every image
  uint32_t skey[kSortThreads];
  uint32_t sidx[kSortThreads];
  int before, all;
};
__device__ __noinline__ void det_select_slowly(
    const float* __restrict__ conf, const DBox* __restrict__ boxes, int P, int C, int loc_classes,
    int keep_top_k, int max_cand, const int* __restrict__ kept_idx, const int* s_off, int total,
    int i, float* __restrict__ rows_image, int* __restrict__ rows_count,
    int* __restrict__ cut_tie_flag, SelectShortLds* st) {
  select_short(conf, boxes, P, C, loc_classes, keep_top_k, max_cand, kept_idx, s_off, total, i,
               rows_image, rows_count, cut_tie_flag, st);
}
__global__ __launch_bounds__(kSortThreads) void det_select_fast_kernel(
    const float* __restrict__ conf, const DBox* __restrict__ boxes, int P, int loc_classes,
    const int* __restrict__ kept_idx, const uint32_t* __restrict__ kept_key,
    const DBox* __restrict__ kept_box, const int* __restrict__ kept_count, int num, int C,
    int max_cand, int keep_top_k, float* __restrict__ rows_tmp, int* __restrict__ rows_count,
    int max_rows, float* __restrict__ out, int* __restrict__ num_rows,
    int* __restrict__ cut_tie_flag) {
  __shared__ SelectFastLds lds;
  __shared__ SelectShortLds short_lds;
  __shared__ int s_off[1024];
  const int i = blockIdx.x, tid = threadIdx.x;
  for (int t = tid; t < num; t += kSortThreads) lds.rows[t] = 0;
  __syncthreads();
  for (int t = tid; t < num * C; t += kSortThreads) atomicAdd(&lds.rows[t / C], kept_count[t]);
  for (int c = tid; c < C; c += kSortThreads) s_off[c + 1] = kept_count[i * C + c];
  __syncthreads();
  if (tid < 64) {
    int before = 0, all = 0;
    for (int t = tid; t < num; t += 64) {
      int r = lds.rows[t];
      if (keep_top_k > -1 && r > keep_top_k) r = keep_top_k;
      all += r;
      if (t < i) before += r;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      before += __shfl_xor(before, o, 64);
      all += __shfl_xor(all, o, 64);
    }
    if (tid == 0) {
      lds.before = before;
      lds.all = all;
      int off = 0;
      for (int c = 0; c < C; ++c) {
        const int cnt = s_off[c + 1];
        s_off[c] = off;
        off += cnt;
      }
      s_off[C] = off;
    }
  }
  __syncthreads();
  const int all = lds.all, before = lds.before, total = s_off[C];
  if (all == 0) {
    // one row of -1 per image carrying the image index (detection_output_layer.cpp:175-185)
    if (i == 0) {
      for (int t = tid; t < num * 7 && t < max_rows * 7; t += kSortThreads)
        out[t] = (t % 7 == 0) ? static_cast<float>(t / 7) : -1.f;
      if (tid == 0) *num_rows = num;
    }
    return;
  }
  if (i == 0 && tid == 0) *num_rows = all < max_rows ? all : max_rows;
  // entry e of the image = (label, place in that label's NMS order), labels ascending
  auto label_of = [&](int e) {
    int lo = 0, hi = C - 1;  // the last label whose entries start at or before e
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (s_off[mid] <= e) lo = mid; else hi = mid - 1;
    }
    // (labels without entries share their start with the next one: step over them)
    while (s_off[lo + 1] <= e) ++lo;
    return lo;
  };
  auto write_row = [&](int row, int e, int c) {
    if (before + row >= max_rows) return;
    const size_t at = (size_t)(i * C + c) * max_cand + (e - s_off[c]);
    const uint32_t asc = ~kept_key[at];
    const float score = __uint_as_float((asc & 0x80000000u) ? (asc & 0x7fffffffu) : ~asc);
    const DBox b = kept_box[at];
    float* r = out + (size_t)(before + row) * 7;
    r[0] = static_cast<float>(i);
    r[1] = static_cast<float>(c);
    r[2] = score;
    r[3] = b.xmin;
    r[4] = b.ymin;
    r[5] = b.xmax;
    r[6] = b.ymax;
  };
  if (keep_top_k < 0 || total <= keep_top_k) {
    for (int e = tid; e < total; e += kSortThreads) write_row(e, e, label_of(e));
    return;
  }
  uint32_t key = 0xffffffffu, e_sel = 0xffffffffu;
  int m = 0;
  // Every label's list is in descending score order, so the image's best entries sit at the
  // heads of the lists.  First the heads alone: R entries of every label, one to a thread,
  // ordered by the compare-exchange network.  If no list that goes on behind its head has
  // its R-th entry at or below the keep_top_k-th key of the heads, nothing further down any
  // list can be among the best keep_top_k (or tie with the last of them), and the heads hold
  // the answer.  A label with more than R of the best entries sends the image to the
  // selection over all entries below, which then starts from the heads' cut.
  uint32_t cut = 0;  // the heads' keep_top_k-th key when the heads did not settle it: the true one is no larger
  const int R = kSortThreads / C;
  if (R >= 1) {  // uniform
    const int c = tid / R, r = tid - c * R;
    const int cnt = c < C ? s_off[c + 1] - s_off[c] : 0;
    if (r < cnt) {
      key = kept_key[(size_t)(i * C + c) * max_cand + r];
      e_sel = static_cast<uint32_t>(s_off[c] + r);
    }
    const uint32_t head_end = (r == R - 1 && cnt > R) ? key : 0xffffffffu;
    bitonic_sort_block<kSortThreads>(key, e_sel, lds.sel.x, lds.sel.x + kSortThreads);
    __syncthreads();
    if (tid == keep_top_k - 1) lds.sel.x[0] = key;
    __syncthreads();
    const uint32_t tau = lds.sel.x[0];
    // (tau all ones: the heads hold fewer than keep_top_k entries)
    if (!__syncthreads_or(tau == 0xffffffffu || head_end <= tau))
      m = __syncthreads_count(key <= tau);
    else if (tau != 0xffffffffu)
      cut = tau;
  }
  if (m == 0) {  // uniform
    uint32_t rk[kSelLdsPer];
    int c = label_of(min(tid, total - 1));  // a thread's entries ascend: so do their labels
#pragma unroll
    for (int j = 0; j < kSelLdsPer; ++j) {
      const int e = tid + j * kSortThreads;
      rk[j] = 0xffffffffu;
      if (e < total) {
        while (s_off[c + 1] <= e) ++c;
        rk[j] = kept_key[(size_t)(i * C + c) * max_cand + (e - s_off[c])];
      }
    }
    m = block_select_smallest<kSelLdsPer>(rk, keep_top_k, &lds.sel, &key, &e_sel, cut);
  }
  if (m == 0) {  // uniform
    float* tmp = rows_tmp + (size_t)i * C * max_cand * 7;
    det_select_slowly(conf, boxes, P, C, loc_classes, keep_top_k, max_cand, kept_idx, s_off, total, i,
                      tmp, rows_count, cut_tie_flag, &short_lds);
    __threadfence_block();
    __syncthreads();
    for (int t = tid; t < keep_top_k * 7; t += kSortThreads)
      if (before + t / 7 < max_rows) out[(size_t)before * 7 + t] = tmp[t];
    return;
  }
  // thread t < keep_top_k holds the entry of rank t by (score, entry); its row is its rank
  // by entry among those
  const bool mine = tid < keep_top_k;
  lds.skey[tid] = key;
  lds.sidx[tid] = mine ? e_sel : 0xffffffffu;
  __syncthreads();
  if (cut_tie_flag) {
    // more entries at the cut's score than places: which of them survive is decided here by
    // entry order and in the reference by std::sort's internals
    if (tid == 0 && m > keep_top_k) atomicOr(cut_tie_flag, 1);
    // equal scores of one label among the kept rows (neighbours in this order: equal scores
    // are ordered by entry, and a label's entries are contiguous): the reference rebuilds
    // the label's list in std::sort's order, here they stay in NMS order
    if (mine && tid + 1 < keep_top_k && lds.skey[tid + 1] == key &&
        label_of(static_cast<int>(lds.sidx[tid + 1])) == label_of(static_cast<int>(e_sel)))
      atomicOr(cut_tie_flag, 2);
  }
  if (mine) {
    int row = 0;
    for (int t = 0; t < keep_top_k; ++t) row += lds.sidx[t] < e_sel;
    write_row(row, static_cast<int>(e_sel), label_of(static_cast<int>(e_sel)));
  }
}

// Concatenates the per-image rows, one workgroup per image; with no detection at
// all, one row of -1 per image carrying the image index
// (detection_output_layer.cpp:175-185).
__global__ __launch_bounds__(256) void det_emit_kernel(const float* __restrict__ rows_tmp,
                                                       const int* __restrict__ rows_count,
                                                       int num, int max_entries, int max_rows,
                                                       float* __restrict__ out,
                                                       int* __restrict__ num_rows) {
  __shared__ int s_before, s_total;
  const int i = blockIdx.x;
  if (threadIdx.x < 64) {
    // rows of the images before this one, and of all
    int before = 0, total = 0;
    for (int k = threadIdx.x; k < num; k += 64) {
      const int c = rows_count[k];
      total += c;
      if (k < i) before += c;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      before += __shfl_xor(before, o, 64);
      total += __shfl_xor(total, o, 64);
    }
    if (threadIdx.x == 0) {
      s_before = before;
      s_total = total;
    }
  }
  __syncthreads();
  const int total = s_total;
  if (total == 0) {
    if (i == 0) {
      for (int t = threadIdx.x; t < num * 7 && t < max_rows * 7; t += 256)
        out[t] = (t % 7 == 0) ? static_cast<float>(t / 7) : -1.f;
      if (threadIdx.x == 0) *num_rows = num;
    }
    return;
  }
  const int cnt = rows_count[i], off = s_before;
  const float* src = rows_tmp + (size_t)i * max_entries * 7;
  float* dst = out + (size_t)off * 7;
  for (int t = threadIdx.x; t < cnt * 7; t += 256)
    if (off + t / 7 < max_rows) dst[t] = src[t];
  if (i == 0 && threadIdx.x == 0) *num_rows = total < max_rows ? total : max_rows;
}

struct DetLayout {
  size_t boxes, k0, v0, k1, v1, kept_idx, kept_count, sk0, sv0, sk1, sv1, selected, rows_tmp,
      rows_count, cand_key, cand_idx, cand_box, ncand, col_rejects, kept_key, kept_box, total;
};

inline size_t det_align(size_t v) { return (v + 255) / 256 * 256; }

DetLayout det_layout(int num, int P, int C, int loc_classes, int max_cand) {
  DetLayout L;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    const size_t at = off;
    off += det_align(bytes);
    return at;
  };
  const size_t segs = (size_t)num * C;
  const size_t entries = (size_t)num * C * max_cand;
  L.boxes = take(sizeof(DBox) * (size_t)num * loc_classes * P);
  L.k0 = take(4 * segs * P);
  L.v0 = take(4 * segs * P);
  L.k1 = take(4 * segs * P);
  L.v1 = take(4 * segs * P);
  L.kept_idx = take(4 * entries);
  L.kept_count = take(4 * segs);
  L.sk0 = take(4 * entries);
  L.sv0 = take(4 * entries);
  L.sk1 = take(4 * entries);
  L.sv1 = take(4 * entries);
  L.selected = take(4 * entries);
  L.rows_tmp = take(4 * 7 * entries);
  L.rows_count = take(4 * (size_t)num);
  // the three-launch path (top_k <= kDetSplitTopK): candidate lists and their pair bits
  const size_t cands = segs * (size_t)((max_cand + 63) / 64 * 64);
  const bool split = max_cand <= kDetSplitTopK;
  L.cand_key = take(split ? 4 * cands : 0);
  L.cand_idx = take(split ? 4 * cands : 0);
  L.cand_box = take(split ? sizeof(DBox) * cands : 0);
  L.ncand = take(split ? 4 * segs : 0);
  L.col_rejects = take(split ? 8 * kDetSplitWords * cands : 0);
  L.kept_key = take(split ? 4 * entries : 0);
  L.kept_box = take(split ? sizeof(DBox) * entries : 0);
  L.total = off;
  return L;
}

int det_max_cand(int P, int top_k) { return (top_k > -1 && top_k < P) ? top_k : P; }

// Who takes the three-launch per-class path: 1 = inputs it fits and pays for (tables of
// 4096 priors and more: below that the sort of the whole table in LDS is cheap and one
// launch per class wins, MobileNet-SSD's 32 x 21 lists of 1917 priors 35 against 53 us),
// 2 = every input it fits, 0 = none (test knob).
int g_det_split = 1;

}  // namespace
}  // namespace mchip

using namespace mchip;

extern "C" {

int mcDetectionOutputWorkspaceSize(int num, int num_priors, int num_classes, int share_location,
                                   int top_k, size_t* bytes) {
  MC_REQUIRE(bytes && num > 0 && num_priors > 0 && num_classes > 0,
             "mcDetectionOutputWorkspaceSize: bad argument");
  *bytes = det_layout(num, num_priors, num_classes, share_location ? 1 : num_classes,
                      det_max_cand(num_priors, top_k))
               .total;
  return 0;
}

int mcDetectionOutputMaxRows(int num, int num_priors, int num_classes, int top_k, int keep_top_k) {
  long per_image = (long)num_classes * det_max_cand(num_priors, top_k);
  if (keep_top_k > -1 && keep_top_k < per_image) per_image = keep_top_k;
  long rows = per_image * num;
  if (rows < num) rows = num;
  return rows > 0x7fffffffL ? 0x7fffffff : static_cast<int>(rows);
}

int mcDetectionOutputSplit(int mode) {
  MC_REQUIRE(mode >= 0 && mode <= 2, "mcDetectionOutputSplit: bad argument");
  g_det_split = mode;
  return 0;
}

int mcDetectionOutput(const float* loc, const float* conf, const float* prior, int num,
                      int num_priors, int num_classes, int share_location, int background_label,
                      int code_type, int variance_encoded_in_target, int keep_top_k,
                      float confidence_threshold, float nms_threshold, float eta, int top_k,
                      void* workspace, size_t workspace_bytes, float* out_rows, int max_rows,
                      int* num_rows, int* cut_tie_flag, void* stream) {
  MC_REQUIRE(loc && conf && prior && workspace && out_rows && num_rows,
             "mcDetectionOutput: null argument");
  MC_REQUIRE(num > 0 && num <= 1024 && num_priors > 0 && num_classes > 0 && num_classes < 1024,
             "mcDetectionOutput: bad extents");
  MC_REQUIRE(code_type >= 1 && code_type <= 3, "Unknown LocLossType.");
  // shared locations carry the label -1, which DecodeBBoxesAll then skips as background
  // (bbox_util.cpp:366-371; the layer aborts at detection_output_layer.cpp:122-126)
  MC_REQUIRE(!(share_location && background_label == -1),
             "Could not find location predictions for label -1");
  MC_REQUIRE(nms_threshold >= 0.f, "nms_threshold must be non negative.");
  MC_REQUIRE(eta > 0.f && eta <= 1.f, "eta must be in (0, 1]");
  MC_REQUIRE(max_rows >= num, "mcDetectionOutput: output needs at least one row per image");
  const int loc_classes = share_location ? 1 : num_classes;
  const int max_cand = det_max_cand(num_priors, top_k);
  const DetLayout L = det_layout(num, num_priors, num_classes, loc_classes, max_cand);
  MC_REQUIRE(workspace_bytes >= L.total, "mcDetectionOutput: workspace too small (%zu < %zu)",
             workspace_bytes, L.total);
  char* ws = static_cast<char*>(workspace);
  DBox* boxes = reinterpret_cast<DBox*>(ws + L.boxes);
  auto u32 = [&](size_t off) { return reinterpret_cast<uint32_t*>(ws + off); };
  auto i32 = [&](size_t off) { return reinterpret_cast<int*>(ws + off); };
  hipStream_t st = static_cast<hipStream_t>(stream);
  const long ndec = (long)num * loc_classes * num_priors;
  // constant threshold and at most kDetSplitTopK candidates per class: the per-class work
  // in three launches (candidates, pair bits over the whole chip, scan)
  const bool split = g_det_split != 0 && eta >= 1.f && max_cand <= kDetSplitTopK &&
                     num_priors <= kDetLdsMax && (g_det_split == 2 || num_priors >= 4096);
  det_decode_kernel<<<ceil_div(ndec + (split ? (long)num * num_priors : 0), 256), 256, 0, st>>>(
      loc, prior, num, num_priors, loc_classes, code_type, variance_encoded_in_target, boxes,
      cut_tie_flag, conf, num_classes, split ? u32(L.k0) : nullptr);
  MC_LAUNCH_CHECK();
  if (split) {
    const int cand_stride = (max_cand + 63) / 64 * 64, words = cand_stride / 64;
    DBox* cand_box = reinterpret_cast<DBox*>(ws + L.cand_box);
    unsigned long long* col_rejects = reinterpret_cast<unsigned long long*>(ws + L.col_rejects);
    det_candidates_kernel<<<dim3(num_classes, num), kSortThreads, 0, st>>>(
        u32(L.k0), boxes, num_priors, num_classes, loc_classes, background_label,
        desc_key(confidence_threshold), max_cand, cand_stride, u32(L.cand_key), i32(L.cand_idx),
        cand_box, i32(L.ncand));
    MC_LAUNCH_CHECK();
    det_overlap_kernel<<<dim3(ceil_div(words * (words + 1) / 2, kOverlapWaves), num * num_classes),
                         64 * kOverlapWaves, 0, st>>>(cand_box, i32(L.ncand), cand_stride,
                                                      nms_threshold, col_rejects);
    MC_LAUNCH_CHECK();
    det_scan_kernel<<<num * num_classes, 64, 0, st>>>(
        col_rejects, i32(L.ncand), i32(L.cand_idx), u32(L.cand_key), cand_box, cand_stride, max_cand,
        i32(L.kept_idx), u32(L.kept_key), reinterpret_cast<DBox*>(ws + L.kept_box), i32(L.kept_count));
    MC_LAUNCH_CHECK();
    // (the background label has no entries)
    const int labels = num_classes - (background_label >= 0 && background_label < num_classes ? 1 : 0);
    if (keep_top_k <= kSortThreads && (long)labels * max_cand <= kSelLdsMax) {
      det_select_fast_kernel<<<num, kSortThreads, 0, st>>>(
          conf, boxes, num_priors, loc_classes, i32(L.kept_idx), u32(L.kept_key),
          reinterpret_cast<DBox*>(ws + L.kept_box), i32(L.kept_count), num, num_classes, max_cand,
          keep_top_k, reinterpret_cast<float*>(ws + L.rows_tmp), i32(L.rows_count), max_rows, out_rows,
          num_rows, cut_tie_flag);
      MC_LAUNCH_CHECK();
      return 0;
    }
  } else if (num_priors <= kDetLdsMax)
    det_class_nms_lds_kernel<<<dim3(num_classes, num), kSortThreads, 0, st>>>(
        conf, boxes, num_priors, num_classes, loc_classes, background_label, confidence_threshold,
        nms_threshold, eta, top_k, max_cand, i32(L.kept_idx), i32(L.kept_count));
  else
    det_class_nms_kernel<<<dim3(num_classes, num), kSortThreads, 0, st>>>(
        conf, boxes, num_priors, num_classes, loc_classes, background_label, confidence_threshold,
        nms_threshold, eta, top_k, max_cand, u32(L.k0), i32(L.v0), u32(L.k1), i32(L.v1),
        i32(L.kept_idx), i32(L.kept_count));
  MC_LAUNCH_CHECK();
  det_select_kernel<<<num, kSortThreads, 0, st>>>(
      conf, boxes, num_priors, num_classes, loc_classes, keep_top_k, max_cand, i32(L.kept_idx),
      i32(L.kept_count), u32(L.sk0), i32(L.sv0), u32(L.sk1), i32(L.sv1), i32(L.selected),
      reinterpret_cast<float*>(ws + L.rows_tmp), i32(L.rows_count), cut_tie_flag);
  MC_LAUNCH_CHECK();
  det_emit_kernel<<<num, 256, 0, st>>>(reinterpret_cast<float*>(ws + L.rows_tmp), i32(L.rows_count),
                                     num, num_classes * max_cand, max_rows, out_rows, num_rows);
  MC_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
