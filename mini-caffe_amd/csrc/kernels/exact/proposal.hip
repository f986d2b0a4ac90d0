// Region-proposal tail on the device: anchor decode, top-N ordering, bitmask-IoU
// NMS with a single-wavefront scan, roi gather.  No host round trips: the only
// value that returns to the host is the roi count, which fixes the top's shape.
//
// Restates ProposalLayer::Forward_cpu (reference src/layers/proposal_layer.cpp:261-322);
// replaces GenerataProposalsGPU / NMSKernel / RetrieveRoisGPU and the host-side
// SortBBox + bit scan of the reference's device path (proposal_layer.cu:48-276).
//
// This file is compiled with -ffp-contract=off: the kept-box indices must equal
// the CPU path's bit for bit, so every a*b+c here is two roundings like there.
#include <mutex>
#include <vector>

#include "../mc_common.h"
#include "block_sort.h"
#include "mchip/kernels.h"

namespace mchip {
namespace {

// TransformBBox (proposal_layer.cpp:14-53).  exp() is evaluated in double and
// the product with the extent is narrowed afterwards, as the reference's
// unqualified exp(float) does.
__device__ __forceinline__ float decode_and_clip(float* box, float dx, float dy, float dlw,
                                                 float dlh, float img_w, float img_h,
                                                 float min_size) {
  const float w = box[2] - box[0] + 1;
  const float h = box[3] - box[1] + 1;
  const float ctr_x = box[0] + 0.5f * w;
  const float ctr_y = box[1] + 0.5f * h;
  const float pred_ctr_x = dx * w + ctr_x;
  const float pred_ctr_y = dy * h + ctr_y;
  const float pred_w = static_cast<float>(exp(static_cast<double>(dlw)) * static_cast<double>(w));
  const float pred_h = static_cast<float>(exp(static_cast<double>(dlh)) * static_cast<double>(h));
  box[0] = pred_ctr_x - 0.5f * pred_w;
  box[1] = pred_ctr_y - 0.5f * pred_h;
  box[2] = pred_ctr_x + 0.5f * pred_w;
  box[3] = pred_ctr_y + 0.5f * pred_h;
  box[0] = fmaxf(0.f, fminf(box[0], img_w - 1));
  box[1] = fmaxf(0.f, fminf(box[1], img_h - 1));
  box[2] = fmaxf(0.f, fminf(box[2], img_w - 1));
  box[3] = fmaxf(0.f, fminf(box[3], img_h - 1));
  const float box_w = box[2] - box[0] + 1;
  const float box_h = box[3] - box[1] + 1;
  return (box_w >= min_size && box_h >= min_size) ? 1.f : 0.f;
}

// One thread per proposal, index = (h*W + w)*A + k (proposal_layer.cpp:125-147).
__global__ __launch_bounds__(256) void proposal_decode_kernel(
    const float* __restrict__ fg, const float* __restrict__ bbox, const float* __restrict__ anchors,
    const float* __restrict__ im_info, int A, int H, int W, int feat_stride, float min_size_param,
    float4* __restrict__ boxes, uint32_t* __restrict__ keys, uint32_t* __restrict__ keys_orig,
    int* __restrict__ vals, float* __restrict__ scores, int* __restrict__ flags) {
  const int n = A * H * W;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < 8) flags[i] = 0;  // the call's flag words (nothing reads them before this kernel ends)
  if (i >= n) return;
  const int k = i % A;
  const int pix = i / A;
  const int w = pix % W, h = pix / W;
  const int fm = H * W;
  const float img_h = im_info[0], img_w = im_info[1];
  const float min_size = min_size_param * im_info[2];
  const float x = static_cast<float>(w * feat_stride), y = static_cast<float>(h * feat_stride);
  float box[4] = {x + anchors[k * 4 + 0], y + anchors[k * 4 + 1], x + anchors[k * 4 + 2],
                  y + anchors[k * 4 + 3]};
  const float* b = bbox + h * W + w;
  const float valid = decode_and_clip(box, b[(k * 4 + 0) * fm], b[(k * 4 + 1) * fm],
                                      b[(k * 4 + 2) * fm], b[(k * 4 + 3) * fm], img_w, img_h,
                                      min_size);
  const float s = valid * fg[k * fm + h * W + w];
  boxes[i] = make_float4(box[0], box[1], box[2], box[3]);
  scores[i] = s;
  keys[i] = desc_key(s);
  keys_orig[i] = keys[i];
  vals[i] = i;
}

// Orders all proposals by (score desc, index asc) and flags score ties that
// reach into the first `pre` places.
__global__ __launch_bounds__(kSortThreads) void proposal_sort_kernel(
    uint32_t* k0, int* v0, uint32_t* k1, int* v1, int n, int pre, int* __restrict__ tie_flag,
    const int* __restrict__ skip) {
  if (*skip != 0) return;  // uniform: the head of the table settled the result
  __shared__ BlockSortLds lds;
  block_sort_desc(k0, v0, k1, v1, n, &lds);
  int ties = 0;
  // a tie between two of the first pre+1 keys leaves their order to the
  // reference's quicksort; equal keys <=> equal scores
  for (int i = threadIdx.x; i < pre; i += kSortThreads)
    if (i + 1 < n && k0[i] == k0[i + 1]) ties = 1;
  if (ties) atomicOr(tie_flag, 1);
}

// The same for up to kSortLdsMax proposals, sorted inside LDS.
constexpr int kSortLdsPer = 44;
constexpr int kSortLdsMax = kSortLdsPer * kSortThreads;  // 22528
__global__ __launch_bounds__(kSortThreads) void proposal_sort_lds_kernel(
    uint32_t* k0, int* v0, int n, int pre, int* __restrict__ tie_flag,
    const int* __restrict__ skip) {
  if (*skip != 0) return;  // uniform: the head of the table settled the result
  __shared__ BlockSortLds16 lds;
  __shared__ uint32_t s_key[kSortLdsMax];
  __shared__ unsigned short s_val[kSortLdsMax];
  for (int i = threadIdx.x; i < n; i += kSortThreads) {
    s_key[i] = k0[i];
    s_val[i] = static_cast<unsigned short>(i);  // v0[i] == i on entry
  }
  __syncthreads();
  // (foreground probabilities of a two-class softmax spread over many exponents)
  block_sort_desc_lds<kSortLdsPer, unsigned short, false>(s_key, s_val, n, &lds);
  for (int i = threadIdx.x; i < n; i += kSortThreads) {
    k0[i] = s_key[i];
    v0[i] = s_val[i];
  }
  int ties = 0;
  for (int i = threadIdx.x; i < pre; i += kSortThreads)
    if (i + 1 < n && s_key[i] == s_key[i + 1]) ties = 1;
  if (ties) atomicOr(tie_flag, 1);
}

// Boxes and scores of the first `pre` proposals in their final order.
__global__ __launch_bounds__(256) void proposal_order_gather_kernel(
    const int* __restrict__ order, int pre, const float4* __restrict__ boxes,
    const float* __restrict__ scores, float4* __restrict__ sorted_boxes,
    float* __restrict__ sorted_scores, const int* __restrict__ skip) {
  if (skip != nullptr && *skip != 0) return;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= pre) return;
  const int src = order[i];
  sorted_boxes[i] = boxes[src];
  sorted_scores[i] = scores[src];
}

// ---- the head of the table first ---------------------------------------------------
//
// The greedy pass stops at post_nms_topn kept boxes, usually a few hundred candidates
// into the table (config 4: the 300th kept box is candidate 461 of 6000), so ordering
// all proposals, and replaying the reference's order of equal scores over all of
// them, is mostly work whose result nobody reads.  The first step therefore orders
// only the best `want` proposals (one super-block of the scan): the want-th best score
// is found by bisection on the key bits, the proposals at or above it are compacted in
// index order and sorted by (score descending, index ascending).  The scan over them
// either reaches post_nms_topn kept boxes, or the full-size path behind it starts over.
//
// Equal scores: SortBBox (proposal_layer.cpp:88-111) leaves them in an order of its own,
// which only the replay kernels below know.  It cannot matter when, of the proposals
// that share a score, at most one is still alive when the scan reaches them (alive:
// overlaps no box kept before the group): the others are dropped wherever they stand,
// the live one is kept wherever it stands, and the kept sequence is the same for every
// order of the group.  proposal_head_check_kernel verifies exactly that for every group
// of equal scores the scan reached (a group that hangs over the end of the head, where
// the order would also decide who is in, counts as not settled), and only then reports
// the result as complete.
constexpr int kHeadWant = 512;                        // = kScanRows, one super-block of the scan
constexpr int kHeadThreads = kSortThreads;
constexpr int kHeadPer = 44;                          // keys per thread
constexpr int kHeadMaxN = kHeadPer * kHeadThreads;    // 22528 proposals

// info[0] = number of ordered entries m >= want (the keys at or below the want-th smallest),
// 0 when the head could not be ordered here (more candidates than the kernel holds: equal
// scores in crowds; the full-size path takes over).  out_keys / out_order[0 .. m): (key
// ascending = score descending, index ascending); the boxes and scores of the first
// `want` of them go to sorted_boxes / sorted_scores.
__global__ __launch_bounds__(kHeadThreads) void proposal_head_kernel(
    const uint32_t* __restrict__ keys, int n, int want, uint32_t* __restrict__ out_keys,
    int* __restrict__ out_order, int* __restrict__ info, const float4* __restrict__ boxes,
    const float* __restrict__ scores, float4* __restrict__ sorted_boxes,
    float* __restrict__ sorted_scores) {
  __shared__ BlockSelectLds sel;
  const int tid = threadIdx.x;
  // any thread may hold any key: coalesced loads, key i in thread i % threads (no branches
  // around the loads: all of them are in flight together)
  uint32_t rk[kHeadPer];
#pragma unroll
  for (int j = 0; j < kHeadPer; ++j) rk[j] = keys[min(tid + j * kHeadThreads, n - 1)];
  __builtin_amdgcn_sched_barrier(0);  // (or each load is waited for before the next is issued)
#pragma unroll
  for (int j = 0; j < kHeadPer; ++j)
    rk[j] = tid + j * kHeadThreads < n ? min(rk[j], 0xfffffffeu) : 0xffffffffu;  // (all ones: no entry)
  uint32_t key, idx;
  const int m = block_select_smallest<kHeadPer>(rk, want, &sel, &key, &idx);
  if (m == 0) {  // uniform
    if (tid == 0) info[0] = 0;
    return;
  }
  if (tid < m) {
    out_keys[tid] = key;
    out_order[tid] = static_cast<int>(idx);
  }
  if (tid < want) {
    sorted_boxes[tid] = boxes[idx];
    sorted_scores[tid] = scores[idx];
  }
  if (tid == 0) info[0] = m;
}

// After the scan over the head: is its result the whole layer's?  flags[2] (done): the
// scan settled (post_nms_topn kept boxes, or the head was the whole table); flags[3]
// (complete) is set when, besides, no group of equal scores that the scan reached has two
// live members or hangs over the end of the head.  Otherwise done is cleared again and
// the full-size path behind this kernel runs.  mask: rows of the head corner, `stride`
// words each.
__global__ __launch_bounds__(512) void proposal_head_check_kernel(
    const uint32_t* __restrict__ head_keys, const int* __restrict__ info, int want,
    const int* __restrict__ kept, const int* __restrict__ num_kept, int max_keep,
    const unsigned long long* __restrict__ mask, int stride, int* __restrict__ flags,
    const float4* __restrict__ sorted_boxes, const float* __restrict__ sorted_scores,
    float* __restrict__ rois, float* __restrict__ roi_scores, int* __restrict__ state) {
  __shared__ unsigned char alive[kHeadWant];
  __shared__ int s_need;
  const int z = threadIdx.x;
  const int m = info[0];
  const int count = *num_kept;
  if (z == 0) s_need = (m == 0 || flags[2] == 0) ? 1 : 0;
  // the last candidate the scan examined
  const int last = count >= max_keep ? kept[max_keep - 1] : want - 1;
  bool member = false;
  int first = z;
  if (z < kHeadWant) alive[z] = 0;
  if (m > 0 && z < want) {
    const uint32_t k = head_keys[z];
    member = (z > 0 && head_keys[z - 1] == k) || (z + 1 < m && head_keys[z + 1] == k);
    if (member) {
      while (first > 0 && head_keys[first - 1] == k) --first;
      bool live = true;
      if (first <= last) {
        for (int r = 0; r < count && live; ++r) {
          const int kb = kept[r];
          if (kb >= first) break;  // kept[] ascends
          live = !((mask[static_cast<size_t>(kb) * stride + (z >> 6)] >> (z & 63)) & 1ull);
        }
      }
      alive[z] = live ? 1 : 0;
    }
  }
  __syncthreads();
  if (member && first == z && z <= last) {
    // this thread owns the group that starts here
    const uint32_t k = head_keys[z];
    int live = 0, end = z;
    while (end < want && end < m && head_keys[end] == k) live += alive[end++];
    // more of the group beyond the head (which is also the table's cut when the head is all of it)
    const bool hangs_over = end == want && end < m && head_keys[end] == k;
    if (live >= 2 || hangs_over) s_need = 1;
  }
  __syncthreads();
  const int complete = s_need ? 0 : 1;
  if (z == 0) {
    flags[3] = complete;
    if (!complete) flags[2] = 0;
    if (state != nullptr) {  // (the step was called by itself)
      state[0] = 0;
      state[1] = complete;
    }
  }
  // rois[r] = (0, x1, y1, x2, y2) of the r-th kept box (proposal_layer.cpp:187-203); the
  // head holds at most 512 kept boxes
  if (complete && z < count) {
    const float4 b = sorted_boxes[kept[z]];
    rois[z * 5 + 0] = 0.f;
    rois[z * 5 + 1] = b.x;
    rois[z * 5 + 2] = b.y;
    rois[z * 5 + 3] = b.z;
    rois[z * 5 + 4] = b.w;
    if (roi_scores) roi_scores[z] = sorted_scores[kept[z]];
  }
}

// Exact replay of the reference's SortBBox (proposal_layer.cpp:88-111) for inputs
// with equal scores, where the final order is whatever that quicksort leaves.
//
// The recursion is replayed level by level: all partitions of one depth at once.
// A partition with pivot K = a[lo] never moves elements equal to K; it swaps the
// i-th larger element found from the right (position R_i) with the i-th smaller
// one found from the left (L_i) through a moving hole:
//     a[lo] <- a[R_1],  a[R_i] <- a[L_i],  a[L_i] <- a[R_(i+1)],  pivot -> last hole
// for as long as L_i < R_i (resp. R_(i+1) > L_i).  Ranks come from one prefix
// sum over the whole array, so a level costs a handful of passes regardless of
// how many partitions it holds.  Keys are the order-preserving integer images
// of the scores (smaller key = larger score).  One 1024-thread workgroup; runs
// only when `flag` says ties reach into the first num_top places.
constexpr int kQsThreads = 1024;
constexpr int kQsLds = 7168;  // places the LDS phase can hold (21 bytes each)

__global__ __launch_bounds__(kQsThreads) void quicksort_replay_kernel(
    const int* __restrict__ flag, const uint32_t* __restrict__ key_in, int n, int num_top,
    uint32_t* __restrict__ kA, int* __restrict__ vA, uint32_t* __restrict__ kB,
    int* __restrict__ vB, int* __restrict__ seg_lo, int* __restrict__ seg_hi,
    unsigned long long* __restrict__ pref, int* __restrict__ posS, int* __restrict__ posB,
    int* __restrict__ mS, int* __restrict__ mB, int* __restrict__ hole, int* __restrict__ dest,
    int* __restrict__ nseg, unsigned char* __restrict__ cls, int* __restrict__ order_out) {
  if (flag[0] == 0 || flag[1] != 0) return;  // no ties, or tie_replay_fast_kernel did the job
  __shared__ unsigned long long wave_tot[kQsThreads / 64];
  __shared__ int range_lo, range_hi, next_lo, next_hi;
  const int tid = threadIdx.x;
  // Phases that only need "every element once" walk the array with a stride of
  // the workgroup size (coalesced, iterations independent so loads overlap);
  // the prefix sum needs contiguous per-thread runs.  A position whose segment
  // is finished (or lies wholly beyond num_top) is final: its index is written
  // to order_out then, and later levels only walk [range_lo, range_hi], the
  // span of the segments still open, which shrinks to about num_top places
  // after the first few levels.
  for (int p = tid; p < n; p += kQsThreads) {
    kA[p] = key_in[p];
    vA[p] = p;
    seg_lo[p] = 0;
    seg_hi[p] = n - 1;
  }
  if (tid == 0) {
    range_lo = 0;
    range_hi = n - 1;
  }
  __syncthreads();
  uint32_t* __restrict__ key = kA;
  int* __restrict__ val = vA;
  uint32_t* __restrict__ nkey = kB;
  int* __restrict__ nval = vB;
  bool open_left = true;
  for (;;) {
    const int r0 = range_lo, r1 = range_hi + 1;  // open span [r0, r1)
    if (r1 - r0 <= kQsLds && n <= 65535) break;  // small enough to finish in LDS
    const int per = (r1 - r0 + kQsThreads - 1) / kQsThreads;
    const int begin = min(r0 + tid * per, r1), end = min(begin + per, r1);
    if (tid == 0) {
      next_lo = n;
      next_hi = -1;
    }
    // 1. classify against the segment's pivot: 1 = smaller score, 2 = larger score
#pragma unroll 12
    for (int p = r0 + tid; p < r1; p += kQsThreads) {
      const int lo = seg_lo[p];
      unsigned char f = 0;
      if (lo >= 0 && p != lo) {
        const uint32_t K = key[lo], k = key[p];
        f = k > K ? 1 : (k < K ? 2 : 0);
      }
      if (lo == p) {
        mS[p] = 0;
        mB[p] = 0;
      }
      cls[p] = f;
      dest[p] = p;
    }
    __syncthreads();
    // inclusive prefix counts over the open span (smaller: low word, larger: high word)
    unsigned long long local = 0;
    for (int p = begin; p < end; ++p) {
      const unsigned char f = cls[p];
      local += f == 1 ? 1ull : (f == 2 ? (1ull << 32) : 0ull);
    }
    unsigned long long inc = local;
    {
      const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const unsigned lo32 = __shfl_up(static_cast<unsigned>(inc), o, 64);
        const unsigned hi32 = __shfl_up(static_cast<unsigned>(inc >> 32), o, 64);
        if (lane >= o) inc += (static_cast<unsigned long long>(hi32) << 32) | lo32;
      }
      if (lane == 63) wave_tot[wave] = inc;
      __syncthreads();
      unsigned long long base = 0;
      for (int w = 0; w < wave; ++w) base += wave_tot[w];
      inc = base + inc - local;  // exclusive prefix of this thread's run
    }
    for (int p = begin; p < end; ++p) {
      const unsigned char f = cls[p];
      inc += f == 1 ? 1ull : (f == 2 ? (1ull << 32) : 0ull);
      pref[p] = inc;
    }
    __syncthreads();
    // 2. rank -> position tables
#pragma unroll 12
    for (int p = r0 + tid; p < r1; p += kQsThreads) {
      const unsigned char f = cls[p];
      if (f == 0) continue;
      const int lo = seg_lo[p];
      const unsigned long long base = pref[lo], mine = pref[p];
      if (f == 1) {
        posS[lo + static_cast<int>((mine & 0xffffffffull) - (base & 0xffffffffull))] = p;
      } else {
        const int nB = static_cast<int>((pref[seg_hi[p]] >> 32) - (base >> 32));
        posB[lo + nB - static_cast<int>((mine >> 32) - (base >> 32)) + 1] = p;
      }
    }
    __syncthreads();
    // 3. who moves where
#pragma unroll 12
    for (int p = r0 + tid; p < r1; p += kQsThreads) {
      const unsigned char f = cls[p];
      if (f == 0) continue;
      const int lo = seg_lo[p];
      const unsigned long long base = pref[lo], top = pref[seg_hi[p]], mine = pref[p];
      const int nS = static_cast<int>((top & 0xffffffffull) - (base & 0xffffffffull));
      const int nB = static_cast<int>((top >> 32) - (base >> 32));
      if (f == 1) {
        const int i = static_cast<int>((mine & 0xffffffffull) - (base & 0xffffffffull));
        if (i <= nB && p < posB[lo + i]) {
          dest[p] = posB[lo + i];
          const int nx = i + 1;
          if (!(nx <= nS && nx <= nB && posS[lo + nx] < posB[lo + nx])) mS[lo] = i;
        }
      } else {
        const int i = nB - static_cast<int>((mine >> 32) - (base >> 32)) + 1;
        if (i == 1 || (i - 1 <= nS && p > posS[lo + i - 1])) {
          dest[p] = i == 1 ? lo : posS[lo + i - 1];
          const int nx = i + 1;
          if (!(nx <= nB && nx - 1 <= nS && posB[lo + nx] > posS[lo + nx - 1])) mB[lo] = i;
        }
      }
    }
    __syncthreads();
    // 4. pivots find the final hole; an all-equal segment is final as it stands
#pragma unroll 12
    for (int p = r0 + tid; p < r1; p += kQsThreads) {
      if (seg_lo[p] != p) continue;
      const bool all_equal = pref[seg_hi[p]] == pref[p];
      int h;
      if (mB[p] == 0) h = p;
      else if (mB[p] > mS[p]) h = posB[p + mB[p]];
      else h = posS[p + mS[p]];
      hole[p] = all_equal ? -1 : h;
      dest[p] = h;
    }
    __syncthreads();
    // 5. apply the moves, derive the next level's segments; a place that stays
    // open is carried to the other buffer, a place that closes is final
    int my_lo = n, my_hi = -1;
#pragma unroll 12
    for (int p = r0 + tid; p < r1; p += kQsThreads) {
      const int lo = seg_lo[p];
      if (lo < 0) {  // closed on an earlier level (inside the span, between open segments)
        nseg[2 * p] = -1;
        nseg[2 * p + 1] = -1;
        continue;
      }
      const int d = dest[p];
      const int hi = seg_hi[p];
      const int h = hole[lo];
      // the segment the element's NEW place d belongs to on the next level
      int nlo = -1, nhi = -1;
      if (h >= 0) {
        if (d < h) {
          if (lo < h - 1) {
            nlo = lo;
            nhi = h - 1;
          }
        } else if (d > h) {
          if (h + 1 < num_top && h + 1 < hi) {
            nlo = h + 1;
            nhi = hi;
          }
        }
      }
      if (nlo >= 0) {
        nkey[d] = key[p];
        nval[d] = val[p];
        my_lo = min(my_lo, nlo);
        my_hi = max(my_hi, nhi);
      } else if (d < num_top) {
        order_out[d] = val[p];
      }
      nseg[2 * d] = nlo;
      nseg[2 * d + 1] = nhi;
    }
    if (my_hi >= 0) {
      atomicMin(&next_lo, my_lo);
      atomicMax(&next_hi, my_hi);
    }
    __syncthreads();
#pragma unroll 12
    for (int p = r0 + tid; p < r1; p += kQsThreads) {
      seg_lo[p] = nseg[2 * p];
      seg_hi[p] = nseg[2 * p + 1];
    }
    uint32_t* tk = key; key = nkey; nkey = tk;
    int* tv = val; val = nval; nval = tv;
    const int nh = next_hi, nl = next_lo;
    __syncthreads();
    if (nh < 0) {
      open_left = false;
      break;
    }
    if (tid == 0) {
      range_lo = nl;
      range_hi = nh;
    }
    __syncthreads();
  }
  if (!open_left) return;

  // ---- the same levels with every per-place array in LDS -------------------
  // Places are counted from `base`; 0xFFFF marks a closed place.  Per-pivot
  // values live in otherwise unused slots: the counts of moved elements in
  // slot 0 of the pivot's rank tables (ranks start at 1), the hole in the
  // pivot's own dest, "all equal" as class 3 of the pivot.  Keys and indices
  // are permuted in place: each thread reads its places, the workgroup
  // synchronises, each thread writes them to their destinations.
  __shared__ unsigned short s_lo[kQsLds], s_hi[kQsLds], s_posS[kQsLds], s_posB[kQsLds],
      s_dest[kQsLds], s_val[kQsLds];
  __shared__ unsigned char s_cls[kQsLds];
  __shared__ uint32_t s_pref[kQsLds], s_key[kQsLds];
  constexpr unsigned short kClosed = 0xFFFF;
  constexpr int kPerThread = (kQsLds + kQsThreads - 1) / kQsThreads;
  const int base = range_lo;
  {
    const int span = range_hi + 1 - base;
    for (int q = tid; q < span; q += kQsThreads) {
      const int lo = seg_lo[base + q];
      s_lo[q] = lo < 0 ? kClosed : static_cast<unsigned short>(lo - base);
      s_hi[q] = lo < 0 ? kClosed : static_cast<unsigned short>(seg_hi[base + q] - base);
      s_key[q] = key[base + q];
      s_val[q] = static_cast<unsigned short>(val[base + q]);
    }
  }
  __syncthreads();
  if (tid == 0) {
    range_lo = 0;
    range_hi = range_hi - base;
  }
  __syncthreads();
  for (;;) {
    const int r0 = range_lo, r1 = range_hi + 1;
    const int per = (r1 - r0 + kQsThreads - 1) / kQsThreads;
    const int begin = min(r0 + tid * per, r1), end = min(begin + per, r1);
    if (tid == 0) {
      next_lo = kQsLds;
      next_hi = -1;
    }
    // 1. classify
    for (int q = r0 + tid; q < r1; q += kQsThreads) {
      const unsigned short lo = s_lo[q];
      unsigned char f = 0;
      if (lo != kClosed && q != lo) {
        const uint32_t K = s_key[lo], k = s_key[q];
        f = k > K ? 1 : (k < K ? 2 : 0);
      }
      if (lo == q) {
        s_posS[q] = 0;  // moved smaller-score elements of this pivot's partition
        s_posB[q] = 0;  // moved larger-score elements
      }
      s_cls[q] = f;
      s_dest[q] = static_cast<unsigned short>(q);
    }
    __syncthreads();
    // prefix counts: smaller in the low half, larger in the high half
    uint32_t local = 0;
    for (int q = begin; q < end; ++q) {
      const unsigned char f = s_cls[q];
      local += f == 1 ? 1u : (f == 2 ? (1u << 16) : 0u);
    }
    uint32_t inc = local;
    {
      const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const uint32_t up = __shfl_up(inc, o, 64);
        if (lane >= o) inc += up;
      }
      if (lane == 63) wave_tot[wave] = inc;
      __syncthreads();
      uint32_t before = 0;
      for (int w = 0; w < wave; ++w) before += static_cast<uint32_t>(wave_tot[w]);
      inc = before + inc - local;
    }
    for (int q = begin; q < end; ++q) {
      const unsigned char f = s_cls[q];
      inc += f == 1 ? 1u : (f == 2 ? (1u << 16) : 0u);
      s_pref[q] = inc;
    }
    __syncthreads();
    // 2. rank -> place tables
    for (int q = r0 + tid; q < r1; q += kQsThreads) {
      const unsigned char f = s_cls[q];
      if (f == 0) continue;
      const int lo = s_lo[q];
      const uint32_t b = s_pref[lo], mine = s_pref[q];
      if (f == 1) {
        s_posS[lo + static_cast<int>((mine & 0xffffu) - (b & 0xffffu))] = static_cast<unsigned short>(q);
      } else {
        const int nB = static_cast<int>((s_pref[s_hi[q]] >> 16) - (b >> 16));
        s_posB[lo + nB - static_cast<int>((mine >> 16) - (b >> 16)) + 1] = static_cast<unsigned short>(q);
      }
    }
    __syncthreads();
    // 3. who moves where.  The moved counts go to slot 0 of the pivot's tables,
    // which this pass never reads (ranks start at 1).
    for (int q = r0 + tid; q < r1; q += kQsThreads) {
      const unsigned char f = s_cls[q];
      if (f == 0) continue;
      const int lo = s_lo[q];
      const uint32_t b = s_pref[lo], top = s_pref[s_hi[q]], mine = s_pref[q];
      const int nS = static_cast<int>((top & 0xffffu) - (b & 0xffffu));
      const int nB = static_cast<int>((top >> 16) - (b >> 16));
      if (f == 1) {
        const int i = static_cast<int>((mine & 0xffffu) - (b & 0xffffu));
        if (i <= nB && q < s_posB[lo + i]) {
          s_dest[q] = s_posB[lo + i];
          const int nx = i + 1;
          if (!(nx <= nS && nx <= nB && s_posS[lo + nx] < s_posB[lo + nx]))
            s_posS[lo] = static_cast<unsigned short>(i);
        }
      } else {
        const int i = nB - static_cast<int>((mine >> 16) - (b >> 16)) + 1;
        if (i == 1 || (i - 1 <= nS && q > s_posS[lo + i - 1])) {
          s_dest[q] = i == 1 ? static_cast<unsigned short>(lo) : s_posS[lo + i - 1];
          const int nx = i + 1;
          if (!(nx <= nB && nx - 1 <= nS && s_posB[lo + nx] > s_posS[lo + nx - 1]))
            s_posB[lo] = static_cast<unsigned short>(i);
        }
      }
    }
    __syncthreads();
    // 4. pivots find the final hole
    for (int q = r0 + tid; q < r1; q += kQsThreads) {
      if (s_lo[q] != q) continue;
      const bool all_equal = s_pref[s_hi[q]] == s_pref[q];
      const int mS_ = s_posS[q], mB_ = s_posB[q];
      int h;
      if (mB_ == 0) h = q;
      else if (mB_ > mS_) h = s_posB[q + mB_];
      else h = s_posS[q + mS_];
      if (all_equal) s_cls[q] = 3;
      s_dest[q] = static_cast<unsigned short>(h);
    }
    __syncthreads();
    // 5. apply: read, synchronise, write
    uint32_t rk[kPerThread];
    unsigned short rv[kPerThread], rd[kPerThread], rlo[kPerThread], rhi[kPerThread];
    int my_lo = kQsLds, my_hi = -1;
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      const int q = r0 + tid + j * kQsThreads;
      rd[j] = kClosed;  // nothing to write
      if (q >= r1) continue;
      const unsigned short lo = s_lo[q];
      if (lo == kClosed) continue;
      const int d = s_dest[q], hi = s_hi[q], h = s_dest[lo];
      const bool all_equal = s_cls[lo] == 3;
      int nlo = -1, nhi = -1;
      if (!all_equal) {
        if (d < h) {
          if (lo < h - 1) {
            nlo = lo;
            nhi = h - 1;
          }
        } else if (d > h) {
          if (base + h + 1 < num_top && h + 1 < hi) {
            nlo = h + 1;
            nhi = hi;
          }
        }
      }
      rk[j] = s_key[q];
      rv[j] = s_val[q];
      rd[j] = static_cast<unsigned short>(d);
      rlo[j] = nlo < 0 ? kClosed : static_cast<unsigned short>(nlo);
      rhi[j] = nlo < 0 ? kClosed : static_cast<unsigned short>(nhi);
      if (nlo >= 0) {
        my_lo = min(my_lo, nlo);
        my_hi = max(my_hi, nhi);
      }
    }
    if (my_hi >= 0) {
      atomicMin(&next_lo, my_lo);
      atomicMax(&next_hi, my_hi);
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      if (rd[j] == kClosed) continue;
      const int d = rd[j];
      s_key[d] = rk[j];
      s_val[d] = rv[j];
      s_lo[d] = rlo[j];
      s_hi[d] = rhi[j];
      if (rlo[j] == kClosed && base + d < num_top) order_out[base + d] = rv[j];
    }
    __syncthreads();
    const int nh = next_hi, nl = next_lo;
    __syncthreads();
    if (nh < 0) break;
    if (tid == 0) {
      range_lo = nl;
      range_hi = nh;
    }
    __syncthreads();
  }
}

// ---- the same replay for inputs with few equal scores ----------------------------
//
// When only a handful of scores are equal (real score maps: a few dozen pairs among
// 20 000), almost every partition of the recursion holds distinct scores only, and for
// such a partition the quicksort's result is simply the sorted order the radix sort has
// already produced.  This kernel therefore follows the recursion only through the
// partitions that still hold (or border on) a pair of equal scores, one partition at a
// time instead of every place of the array on every level:
//   * keys are replaced by their dense rank in sorted order (equal scores, equal rank),
//     so a place is 32 bits, (rank << 16 | original index), and the whole array lives in
//     LDS together with one 16-bit rank -> place table;
//   * sorted places [a, b] are "clean" when no pair of equal neighbours among the sorted
//     keys touches them (one subtraction on a prefix count); a clean child is closed at
//     once, its places keep the radix order;
//   * a partition longer than kFastWaveSeg is done by the whole workgroup, the others by
//     one wavefront each, sixteen at a time.
// A partition about pivot K = a[lo] (proposal_layer.cpp:88-111) as rank arithmetic: the
// i-th smaller score from the left (place L_i) and the i-th larger score from the right
// (R_i) change places through the moving hole while L_i < R_i:
//     a[lo] <- a[R_1],  a[R_i] <- a[L_i],  a[L_i] <- a[R_(i+1)],  pivot -> last hole;
// scores equal to the pivot's never move.  Counts come from wavefront ballots.
// Runs when the radix sort flagged equal scores among the first num_top + 1 and the
// input is small enough; it then sets flag[1] so that quicksort_replay_kernel, which
// handles everything else, returns at once.
constexpr int kFastThreads = 1024;
constexpr int kFastWaves = kFastThreads / 64;
constexpr int kFastMaxN = 22528;          // places held in LDS (6 bytes each)
constexpr int kFastMaxPairs = 500;        // equal neighbour pairs among the first num_top + 1
constexpr int kFastMaxSegs = 2 * kFastMaxPairs + 8;
constexpr int kFastWaveSeg = 512;         // longest partition one wavefront takes
constexpr int kFastChunks = kFastMaxN / 64 + 2;
constexpr int kFastChunksPerWave = (kFastChunks + kFastWaves - 1) / kFastWaves;
constexpr int kFastRegChunks = 8;         // chunks per wavefront whose moved places wait in registers
constexpr int kFastMaxLong = kFastMaxN / kFastWaveSeg + 2;

struct FastLds {
  uint32_t kv[kFastMaxN];                 // (dense rank << 16) | original index, by place
  unsigned short tab[kFastMaxN + 2];      // rank -> place: smaller scores up from lo + 1,
                                          // larger scores down from hi
  unsigned long long ms[kFastChunks], mb[kFastChunks];  // ballots of the workgroup path
  uint32_t cpre[kFastChunks + 1];         // exclusive chunk prefix (smaller low, larger high half)
  uint32_t seg[2][kFastMaxSegs];          // open short partitions (lo << 16 | hi), this level / next
  uint32_t seg_long[2][kFastMaxLong];     // open partitions longer than kFastWaveSeg
  uint32_t wave_cnt[kFastWaves];          // smaller / larger scores in each wavefront's chunks
  unsigned long long pair_bits[kFastChunks];  // bit j: sorted keys j and j + 1 are equal, j < num_top
  unsigned short pair_pre[kFastChunks];       // such pairs in the words before
  int n_pairs;
  int n_seg[2], n_long[2], moved_s, moved_b, failed;
};

// Per-place step shared by both paths.  (ms, mb): ballots of the place's chunk, (ps, pb):
// smaller / larger scores in the chunks before it.  Returns true when the place moves.
struct FastSeg {
  int lo, hi, nS, nB;
};
__device__ __forceinline__ void fast_ranks(const FastSeg& g, unsigned long long ms,
                                           unsigned long long mb, int ps, int pb, int lane,
                                           bool* is_s, bool* is_b, int* rank) {
  const unsigned long long bit = 1ull << lane;
  *is_s = (ms & bit) != 0;
  *is_b = (mb & bit) != 0;
  const unsigned long long lt = bit - 1ull, le = (bit << 1) - 1ull;
  // smaller: rank from the left; larger: rank from the right (both 1-based)
  *rank = *is_s ? ps + __popcll(ms & lt) + 1 : g.nB - (pb + __popcll(mb & le)) + 1;
}

__device__ __forceinline__ bool fast_move(const FastSeg& g, const unsigned short* tab, int q,
                                          bool is_s, bool is_b, int rank, int* dest) {
  if (is_s) {
    if (rank > g.nB) return false;
    const int r = tab[g.hi + 1 - rank];  // R_rank
    *dest = r;
    return q < r;
  }
  if (is_b) {
    if (rank == 1) {
      *dest = g.lo;
      return true;
    }
    if (rank - 1 > g.nS) return false;
    const int l = tab[g.lo + rank - 1];  // L_(rank-1)
    *dest = l;
    return q > l;
  }
  return false;
}

// Pairs of equal neighbours (j, j + 1) of the sorted keys with j < x (counted for j < num_top).
__device__ __forceinline__ int fast_pairs_before(const FastLds* s, int x) {
  const int w = x >> 6;
  return s->pair_pre[w] + __popcll(s->pair_bits[w] & ((1ull << (x & 63)) - 1ull));
}
// True when such a pair touches the sorted places [a, b]: some j in [a - 1, b].
__device__ __forceinline__ bool fast_touched(const FastLds* s, int a, int b) {
  return fast_pairs_before(s, b + 1) - fast_pairs_before(s, max(a - 1, 0)) > 0;
}

// After the moves of a partition: place the pivot, close or queue the two children.
// Called by one thread.
__device__ __forceinline__ void fast_finish(FastLds* s, const FastSeg& g, uint32_t pivot, int u,
                                            int t, int num_top, int* __restrict__ order_out,
                                            int next) {
  const int h = t == 0 ? g.lo : (t > u ? s->tab[g.hi + 1 - t] : s->tab[g.lo + u]);
  if (h < g.lo || h > g.hi || t > g.nB || u > g.nS || (t != u && t != u + 1)) {
    s->failed = 1;  // cannot happen; if it does the general kernel redoes the job
    return;
  }
  s->kv[h] = pivot;
  if (h < num_top) order_out[h] = static_cast<int>(pivot & 0xffffu);
#pragma unroll
  for (int side = 0; side < 2; ++side) {
    const int a = side == 0 ? g.lo : h + 1, b = side == 0 ? h - 1 : g.hi;
    if (a > b) continue;
    if (side == 1 && a >= num_top) continue;  // the reference does not sort past num_top
    if (a == b) {
      if (a < num_top) order_out[a] = static_cast<int>(s->kv[a] & 0xffffu);
      continue;
    }
    if (fast_touched(s, a, b)) {
      const uint32_t entry = (static_cast<uint32_t>(a) << 16) | static_cast<uint32_t>(b);
      if (b - a + 1 > kFastWaveSeg) {
        const int slot = atomicAdd(&s->n_long[next], 1);
        if (slot < kFastMaxLong) s->seg_long[next][slot] = entry;
        else s->failed = 1;
      } else {
        const int slot = atomicAdd(&s->n_seg[next], 1);
        if (slot < kFastMaxSegs) s->seg[next][slot] = entry;
        else s->failed = 1;
      }
    }
  }
}

// Exclusive prefix over up to kFastChunks packed chunk counts (two 16-bit halves) by one
// wavefront: every lane adds up a run of consecutive chunks, one shuffle scan joins the
// runs.  Returns the total in every lane.
__device__ __forceinline__ uint32_t fast_chunk_scan(FastLds* s, int C, int lane) {
  constexpr int kRun = (kFastChunks + 63) / 64;
  uint32_t cnt[kRun], sum = 0;
#pragma unroll
  for (int j = 0; j < kRun; ++j) {
    const int c = lane * kRun + j;
    cnt[j] = c < C ? static_cast<uint32_t>(__popcll(s->ms[c])) |
                         (static_cast<uint32_t>(__popcll(s->mb[c])) << 16)
                   : 0u;
    sum += cnt[j];
  }
  uint32_t inc = sum;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const uint32_t up = __shfl_up(inc, o, 64);
    if (lane >= o) inc += up;
  }
  uint32_t run = inc - sum;
#pragma unroll
  for (int j = 0; j < kRun; ++j) {
    const int c = lane * kRun + j;
    if (c < C) s->cpre[c] = run;
    run += cnt[j];
  }
  return __shfl(inc, 63, 64);
}

__global__ __launch_bounds__(kFastThreads) void tie_replay_fast_kernel(
    int* __restrict__ flag, const uint32_t* __restrict__ sorted_keys, int n, int num_top,
    uint2* __restrict__ stage, int* __restrict__ order) {
  if (flag[0] == 0 || n > kFastMaxN || n < 2) return;
  __shared__ FastLds s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // Equal neighbour pairs of the sorted keys, 64 places per ballot: all of them give the
  // dense ranks, those among the first num_top places are the ones the order depends on.
  {
    const int C = (n + 63) >> 6;
    for (int c = wave; c < C; c += kFastWaves) {
      const int i = (c << 6) + lane;
      const bool eq = i + 1 < n && sorted_keys[i] == sorted_keys[i + 1];
      const unsigned long long all = __ballot(eq), top = __ballot(eq && i < num_top);
      if (lane == 0) {
        s.ms[c] = all;
        s.mb[c] = top;
      }
    }
    __syncthreads();
    if (wave == 0) {
      const uint32_t carry = fast_chunk_scan(&s, C, lane);
      if (lane == 0) {
        s.n_pairs = static_cast<int>(carry >> 16);
        // the whole array, lo 0, hi n - 1, is the first partition
        const bool is_long = n > kFastWaveSeg;
        s.seg[0][0] = s.seg_long[0][0] = static_cast<uint32_t>(n - 1);
        s.n_seg[0] = is_long ? 0 : 1;
        s.n_long[0] = is_long ? 1 : 0;
        s.n_seg[1] = 0;
        s.n_long[1] = 0;
        s.failed = 0;
      }
    }
    __syncthreads();
    if (s.n_pairs > kFastMaxPairs) return;  // uniform: the general kernel runs
    for (int c = wave; c < C; c += kFastWaves) {
      const int i = (c << 6) + lane;
      if (i >= n) continue;
      const unsigned long long lt = (1ull << lane) - 1ull;
      const int before_all = static_cast<int>(s.cpre[c] & 0xffffu) + __popcll(s.ms[c] & lt);
      const int v = order[i];
      s.kv[v] = (static_cast<uint32_t>(i - before_all) << 16) | static_cast<uint32_t>(v);
      if (lane == 0) {
        s.pair_bits[c] = s.mb[c];
        s.pair_pre[c] = static_cast<unsigned short>(s.cpre[c] >> 16);
      }
    }
    if (tid == 0) {  // fast_pairs_before(n) reads one word past the last place when n % 64 == 0
      s.pair_bits[C] = 0;
      s.pair_pre[C] = static_cast<unsigned short>(s.n_pairs);
    }
  }
  __syncthreads();

  // Every level shortens every open partition by at least its pivot: at most n levels.
  int n_cur = s.n_seg[0], n_cur_long = s.n_long[0], cur = 0, levels_left = n + 1;
  __syncthreads();
  while (n_cur + n_cur_long > 0 && levels_left-- > 0) {
    const int next = cur ^ 1;
    // ---- long partitions: the whole workgroup, one after the other ----
    // Every wavefront takes a run of consecutive chunks, so that the counts before a
    // chunk are the wavefront's running sums on top of the totals of the wavefronts
    // before it; ballots are taken again in every pass instead of being stored.
    for (int si = 0; si < n_cur_long; ++si) {
      const uint32_t sg = s.seg_long[cur][si];
      FastSeg g;
      g.lo = static_cast<int>(sg >> 16);
      g.hi = static_cast<int>(sg & 0xffffu);
      const uint32_t pivot = s.kv[g.lo];
      const uint32_t K = pivot >> 16;
      const int places = g.hi - g.lo;  // without the pivot
      const int C = (places + 63) >> 6;
      const int Cw = (C + kFastWaves - 1) / kFastWaves;
      const int c_begin = min(wave * Cw, C), c_end = min(c_begin + Cw, C);
      if (tid == 0) {
        s.moved_s = 0;
        s.moved_b = 0;
      }
      {
        int cs = 0, cb = 0;
        for (int c = c_begin; c < c_end; ++c) {
          const int q = g.lo + 1 + (c << 6) + lane;
          const uint32_t d = q <= g.hi ? s.kv[q] >> 16 : K;
          cs += __popcll(__ballot(d > K));  // larger rank = smaller score
          cb += __popcll(__ballot(d < K));
        }
        if (lane == 0) s.wave_cnt[wave] = static_cast<uint32_t>(cs) | (static_cast<uint32_t>(cb) << 16);
      }
      __syncthreads();
      uint32_t before = 0, total = 0;
#pragma unroll
      for (int w = 0; w < kFastWaves; ++w) {
        const uint32_t v = s.wave_cnt[w];
        before += w < wave ? v : 0u;
        total += v;
      }
      g.nS = static_cast<int>(total & 0xffffu);
      g.nB = static_cast<int>(total >> 16);
      if (g.nS == 0 && g.nB == 0) {
        // every score equals the pivot's: nothing ever moves in here
        for (int q = g.lo + tid; q <= g.hi && q < num_top; q += kFastThreads)
          order[q] = static_cast<int>(s.kv[q] & 0xffffu);
        __syncthreads();  // wave_cnt is reused by the next partition
        continue;
      }
      {
        int ps = static_cast<int>(before & 0xffffu), pb = static_cast<int>(before >> 16);
        for (int c = c_begin; c < c_end; ++c) {
          const int q = g.lo + 1 + (c << 6) + lane;
          const uint32_t d = q <= g.hi ? s.kv[q] >> 16 : K;
          const unsigned long long ms = __ballot(d > K), mb = __ballot(d < K);
          bool is_s, is_b;
          int rank;
          fast_ranks(g, ms, mb, ps, pb, lane, &is_s, &is_b, &rank);
          if (is_s) s.tab[g.lo + rank] = static_cast<unsigned short>(q);
          if (is_b) s.tab[g.hi + 1 - rank] = static_cast<unsigned short>(q);
          ps += __popcll(ms);
          pb += __popcll(mb);
        }
      }
      __syncthreads();
      // A moved place is read by its own lane and written to its destination after
      // every read of the partition is done.  Up to kFastRegChunks chunks per wavefront
      // it waits in registers, in longer partitions (the first few levels) in `stage`.
      int u = 0, t = 0;
      int ps = static_cast<int>(before & 0xffffu), pb = static_cast<int>(before >> 16);
      if (Cw <= kFastRegChunks) {
        uint32_t keep_kv[kFastRegChunks];
        int keep_to[kFastRegChunks];
#pragma unroll
        for (int k = 0; k < kFastRegChunks; ++k) {
          const int c = c_begin + k;
          keep_to[k] = -1;
          if (c < c_end) {
            const int q = g.lo + 1 + (c << 6) + lane;
            const uint32_t mine = q <= g.hi ? s.kv[q] : pivot;
            const uint32_t d = mine >> 16;
            const unsigned long long ms = __ballot(d > K), mb = __ballot(d < K);
            bool is_s, is_b;
            int rank, dest = 0;
            fast_ranks(g, ms, mb, ps, pb, lane, &is_s, &is_b, &rank);
            const bool mv = fast_move(g, s.tab, q, is_s, is_b, rank, &dest);
            if (mv) {
              keep_to[k] = dest;
              keep_kv[k] = mine;
            }
            u += __popcll(__ballot(mv && is_s));
            t += __popcll(__ballot(mv && is_b));
            ps += __popcll(ms);
            pb += __popcll(mb);
          }
        }
        if (lane == 0) {
          if (u) atomicAdd(&s.moved_s, u);
          if (t) atomicAdd(&s.moved_b, t);
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kFastRegChunks; ++k)
          if (keep_to[k] >= 0) s.kv[keep_to[k]] = keep_kv[k];
      } else {
        for (int c = c_begin; c < c_end; ++c) {
          const int q = g.lo + 1 + (c << 6) + lane;
          const uint32_t mine = q <= g.hi ? s.kv[q] : pivot;
          const uint32_t d = mine >> 16;
          const unsigned long long ms = __ballot(d > K), mb = __ballot(d < K);
          bool is_s, is_b;
          int rank, dest = 0;
          fast_ranks(g, ms, mb, ps, pb, lane, &is_s, &is_b, &rank);
          const bool mv = fast_move(g, s.tab, q, is_s, is_b, rank, &dest);
          if (q <= g.hi) stage[q] = make_uint2(mv ? mine : 0u, mv ? static_cast<uint32_t>(dest) : 0xffffffffu);
          u += __popcll(__ballot(mv && is_s));
          t += __popcll(__ballot(mv && is_b));
          ps += __popcll(ms);
          pb += __popcll(mb);
        }
        if (lane == 0) {
          if (u) atomicAdd(&s.moved_s, u);
          if (t) atomicAdd(&s.moved_b, t);
        }
        __syncthreads();
        // every lane reads back what it staged itself, four loads in flight
        for (int c0 = c_begin; c0 < c_end; c0 += 4) {
          uint2 e[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int q = g.lo + 1 + ((c0 + j) << 6) + lane;
            e[j] = (c0 + j < c_end && q <= g.hi) ? stage[q] : make_uint2(0u, 0xffffffffu);
          }
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (e[j].y != 0xffffffffu) s.kv[e[j].y] = e[j].x;
        }
      }
      __syncthreads();
      // One thread places the pivot and queues the children while the others go on to
      // the next partition: it touches the rank table and places of this partition
      // only, and the counters it reads are reset by itself.
      if (tid == 0) fast_finish(&s, g, pivot, s.moved_s, s.moved_b, num_top, order, next);
    }
    // ---- short partitions: one wavefront each ----
    for (int si = wave; si < n_cur; si += kFastWaves) {
      const uint32_t sg = s.seg[cur][si];
      FastSeg g;
      g.lo = static_cast<int>(sg >> 16);
      g.hi = static_cast<int>(sg & 0xffffu);
      const uint32_t pivot = s.kv[g.lo];
      const uint32_t K = pivot >> 16;
      const int places = g.hi - g.lo;
      const int C = (places + 63) >> 6;
      // The wavefront walks the chunks in order, so the counts before a chunk are running
      // sums and nothing but the rank table is stored; the ballots are taken again in
      // every pass (one LDS read and two compares).
      g.nS = 0;
      g.nB = 0;
      for (int c = 0; c < C; ++c) {
        const int q = g.lo + 1 + (c << 6) + lane;
        const uint32_t d = q <= g.hi ? s.kv[q] >> 16 : K;
        g.nS += __popcll(__ballot(d > K));
        g.nB += __popcll(__ballot(d < K));
      }
      if (g.nS == 0 && g.nB == 0) {
        for (int q = g.lo + lane; q <= g.hi && q < num_top; q += 64)
          order[q] = static_cast<int>(s.kv[q] & 0xffffu);
        continue;
      }
      int ps = 0, pb = 0;
      for (int c = 0; c < C; ++c) {
        const int q = g.lo + 1 + (c << 6) + lane;
        const uint32_t d = q <= g.hi ? s.kv[q] >> 16 : K;
        const unsigned long long ms = __ballot(d > K), mb = __ballot(d < K);
        bool is_s, is_b;
        int rank;
        fast_ranks(g, ms, mb, ps, pb, lane, &is_s, &is_b, &rank);
        if (is_s) s.tab[g.lo + rank] = static_cast<unsigned short>(q);
        if (is_b) s.tab[g.hi + 1 - rank] = static_cast<unsigned short>(q);
        ps += __popcll(ms);
        pb += __popcll(mb);
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      int u = 0, t = 0;
      ps = 0;
      pb = 0;
      if (C <= kFastRegChunks) {
        uint32_t keep_kv[kFastRegChunks];
        int keep_to[kFastRegChunks];
#pragma unroll
        for (int c = 0; c < kFastRegChunks; ++c) {
          keep_to[c] = -1;
          if (c < C) {
            const int q = g.lo + 1 + (c << 6) + lane;
            const uint32_t mine = q <= g.hi ? s.kv[q] : pivot;
            const uint32_t d = mine >> 16;
            const unsigned long long ms = __ballot(d > K), mb = __ballot(d < K);
            bool is_s, is_b;
            int rank, dest = 0;
            fast_ranks(g, ms, mb, ps, pb, lane, &is_s, &is_b, &rank);
            const bool mv = fast_move(g, s.tab, q, is_s, is_b, rank, &dest);
            if (mv) {
              keep_to[c] = dest;
              keep_kv[c] = mine;
            }
            u += __popcll(__ballot(mv && is_s));
            t += __popcll(__ballot(mv && is_b));
            ps += __popcll(ms);
            pb += __popcll(mb);
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
        for (int c = 0; c < kFastRegChunks; ++c)
          if (keep_to[c] >= 0) s.kv[keep_to[c]] = keep_kv[c];
      } else {
        for (int c = 0; c < C; ++c) {
          const int q = g.lo + 1 + (c << 6) + lane;
          const uint32_t mine = q <= g.hi ? s.kv[q] : pivot;
          const uint32_t d = mine >> 16;
          const unsigned long long ms = __ballot(d > K), mb = __ballot(d < K);
          bool is_s, is_b;
          int rank, dest = 0;
          fast_ranks(g, ms, mb, ps, pb, lane, &is_s, &is_b, &rank);
          const bool mv = fast_move(g, s.tab, q, is_s, is_b, rank, &dest);
          if (q <= g.hi) stage[q] = make_uint2(mv ? mine : 0u, mv ? static_cast<uint32_t>(dest) : 0xffffffffu);
          u += __popcll(__ballot(mv && is_s));
          t += __popcll(__ballot(mv && is_b));
          ps += __popcll(ms);
          pb += __popcll(mb);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        // every lane reads back what it staged itself, four loads in flight
        for (int c0 = 0; c0 < C; c0 += 4) {
          uint2 e[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int q = g.lo + 1 + ((c0 + j) << 6) + lane;
            e[j] = q <= g.hi ? stage[q] : make_uint2(0u, 0xffffffffu);
          }
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (e[j].y != 0xffffffffu) s.kv[e[j].y] = e[j].x;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      if (lane == 0) fast_finish(&s, g, pivot, u, t, num_top, order, next);
    }
    __syncthreads();
    n_cur = s.failed ? 0 : min(s.n_seg[next], kFastMaxSegs);
    n_cur_long = s.failed ? 0 : min(s.n_long[next], kFastMaxLong);
    if (tid == 0) {  // the lists that were just walked receive the level after next
      s.n_seg[cur] = 0;
      s.n_long[cur] = 0;
    }
    cur = next;
    __syncthreads();
  }
  if (tid == 0 && n_cur + n_cur_long == 0 && !s.failed) {
    flag[1] = 1;
    flag[0] = 3;  // reported to the caller: equal scores, order replayed by this kernel
  }
}

// mask[i][cb] bit j: box cb*64+j (> i) overlaps box i by more than thr, with
// the +1 pixel extents of NonMaximumSuppressionCPU (proposal_layer.cpp:150-185).
// One workgroup of four wavefronts per 64 x 64 tile on or above the diagonal: lane l
// holds column box cb*64 + l, a wavefront takes 16 of the tile's rows (a broadcast
// read each, four independent tests in flight) and a ballot is the row's word.
// The tiles of the upper triangle of `tiles_side` x `tiles_side` blocks are counted row
// by row and dealt to the workgroups of the grid in turn; `nb` = words per row of `mask`.  With `done`: returns at once
// when *done is set.
__global__ __launch_bounds__(256) void nms_mask_kernel(const float4* __restrict__ boxes, int n,
                                                       float thr, int nb, int tiles_side,
                                                       unsigned long long* __restrict__ mask,
                                                       unsigned long long* __restrict__ colmask,
                                                       const int* __restrict__ done) {
  if (done != nullptr && *done != 0) return;  // uniform
  __shared__ float4 rows[64];
  __shared__ unsigned long long cols[64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int total = tiles_side * (tiles_side + 1) / 2;
  for (int t = blockIdx.x; t < total; t += gridDim.x) {
    // tile t of the triangle -> (rb, cb), cb >= rb: row rb starts at rb*side - rb*(rb-1)/2;
    // the largest rb with start(rb) <= t from the quadratic, corrected a step either way
    const float sidef = static_cast<float>(tiles_side) + 0.5f;
    int rb = static_cast<int>(sidef - sqrtf(fmaxf(sidef * sidef - 2.f * static_cast<float>(t), 0.f)));
    rb = max(0, min(rb, tiles_side - 1));
    auto start = [&](int r) { return r * tiles_side - r * (r - 1) / 2; };
    while (rb > 0 && start(rb) > t) --rb;
    while (rb + 1 < tiles_side && start(rb + 1) <= t) ++rb;
    const int cb = rb + (t - start(rb));
    const int rn = min(64, n - rb * 64);
    if (static_cast<int>(threadIdx.x) < rn) rows[threadIdx.x] = boxes[rb * 64 + threadIdx.x];
    const int c = cb * 64 + lane;
    const bool in = c < n;
    const float4 b = boxes[min(c, n - 1)];
    const float area_b = (b.z - b.x + 1) * (b.w - b.y + 1);
    if (threadIdx.x < 64) cols[threadIdx.x] = 0;
    unsigned long long below = 0;  // this lane's column: the earlier boxes of the tile that overlap it
    __syncthreads();
#pragma unroll 1
    for (int r0 = wave * 16; r0 < min(wave * 16 + 16, rn); r0 += 4) {
      unsigned long long bits[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int r = min(r0 + q, rn - 1);
        const float4 a = rows[r];
        const float area_a = (a.z - a.x + 1) * (a.w - a.y + 1);
        const float x1 = fmaxf(a.x, b.x), y1 = fmaxf(a.y, b.y);
        const float x2 = fminf(a.z, b.z), y2 = fminf(a.w, b.w);
        const float w = fmaxf(0.f, x2 - x1 + 1), h = fmaxf(0.f, y2 - y1 + 1);
        const float inter = w * h;
        const float ov = inter / (area_a + area_b - inter);
        const bool hit = in & (c > rb * 64 + r) & (ov > thr);
        bits[q] = __ballot(hit);
        if (hit && r0 + q < rn) below |= 1ull << r;
      }
      if (lane < 4 && r0 + lane < rn)
        mask[static_cast<size_t>(rb * 64 + r0 + lane) * nb + cb] =
            lane == 0 ? bits[0] : lane == 1 ? bits[1] : lane == 2 ? bits[2] : bits[3];
    }
    // A diagonal tile also leaves the transposed words (the overlap is symmetric bit for
    // bit): colmask[c] = the boxes of c's own block before c that overlap it.
    if (colmask != nullptr && rb == cb) {
      if (below) atomicOr(&cols[lane], below);
      __syncthreads();
      if (threadIdx.x < 64 && in) colmask[c] = cols[lane];
    }
    __syncthreads();  // rows and cols are replaced by the next tile's
  }
}

// Greedy scan over the boxes in score order, one workgroup.  The decisions are a
// dependent chain, so nothing on that chain may wait for global memory:
//   * the boxes are taken in super-blocks of kScanBlocks * 64; the part of the
//     mask that relates the boxes of one super-block to each other (64 bytes per
//     box) is staged in LDS; the next super-block's part is fetched into
//     registers while this one is decided and stored once the decisions are done;
//   * wavefront 0 decides: per block of 64 boxes the running "removed" word and
//     the candidates live in scalar registers, so only the boxes that are kept
//     cost an iteration (a lane read of their diagonal word); the rows of kept
//     boxes are folded into the later words of the same super-block from LDS;
//   * after a super-block the whole workgroup folds the rows of its kept boxes
//     into the removed words of all later super-blocks (independent loads, one
//     latency per super-block instead of one per block).
// Words left of the diagonal are never written by nms_mask_kernel and never used.
constexpr int kScanThreads = 512;
constexpr int kScanBlocks = 8;                    // blocks of 64 boxes per super-block
constexpr int kScanRows = kScanBlocks * 64;       // boxes per super-block
constexpr int kScanLoads = kScanRows * kScanBlocks / kScanThreads;  // staged words per thread
static_assert(kHeadWant == kScanRows, "the head is one super-block of the scan");

__device__ inline unsigned long long wave_uniform(unsigned long long v) {
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v >> 32));
  return (static_cast<unsigned long long>(hi) << 32) | lo;
}

// `n` boxes in `nb` blocks; a row of `mask` has `stride` words.  With `done`:
// returns at once when *done is set, and sets it when this scan settles the result
// (`final_part`: the n boxes are all there are; otherwise only if max_keep is reached).
// `resume`: the first super-block was decided by an earlier launch (kept[0 .. *num_kept)
// are its boxes); this one only folds their rows into the later super-blocks and goes on.
__global__ __launch_bounds__(kScanThreads) void nms_scan_kernel(
    const unsigned long long* __restrict__ mask, int n, int nb, int stride, int max_keep,
    int* __restrict__ kept, int* __restrict__ num_kept, int* __restrict__ done, int final_part,
    int resume, const unsigned long long* __restrict__ colmask) {
  extern __shared__ unsigned long long removed[];  // nb words
  __shared__ unsigned long long subcol[kScanRows];  // colmask of the super-block's boxes
  if (done != nullptr && *done != 0) return;  // uniform
  __shared__ unsigned long long sub[kScanRows * kScanBlocks];
  __shared__ int sb_kept[kScanRows];
  __shared__ int s_count, s_ns;
  const int tid = threadIdx.x, lane = tid & 63;
  const bool decider = tid < 64;
  // word `c` of the super-block's row `r`, 0 outside the mask
  auto fetch = [&](int base_blk, int idx) -> unsigned long long {
    const int r = idx / kScanBlocks, c = idx % kScanBlocks;
    const long row = static_cast<long>(base_blk) * 64 + r;
    const int col = base_blk + c;
    return (row < n && col < nb) ? mask[row * stride + col] : 0ull;
  };
  for (int w = tid; w < nb; w += kScanThreads) removed[w] = 0;
  if (resume) {
    const int before = *num_kept;  // at most kScanRows: all from the first super-block
    for (int k = tid; k < before; k += kScanThreads) sb_kept[k] = kept[k];
    if (tid == 0) {
      s_count = before;
      s_ns = before;
    }
  } else {
#pragma unroll
    for (int k = 0; k < kScanLoads; ++k) sub[tid + k * kScanThreads] = fetch(0, tid + k * kScanThreads);
    static_assert(kScanRows == kScanThreads, "one column word per thread");
    subcol[tid] = tid < n ? colmask[tid] : 0ull;
    if (tid == 0) {
      s_count = 0;
      s_ns = 0;
    }
  }
  __syncthreads();
  for (int base_blk = 0; base_blk < nb; base_blk += kScanBlocks) {
    // next super-block's part of the mask, in flight while this one is decided
    unsigned long long ahead[kScanLoads];
    const bool more = base_blk + kScanBlocks < nb;
    if (more) {
#pragma unroll
      for (int k = 0; k < kScanLoads; ++k)
        ahead[k] = fetch(base_blk + kScanBlocks, tid + k * kScanThreads);
    }
    const long next_row = static_cast<long>(base_blk + kScanBlocks) * 64 + tid;
    const unsigned long long ahead_col = (more && next_row < n) ? colmask[next_row] : 0ull;
    if (decider && !(resume && base_blk == 0)) {
      int count = __builtin_amdgcn_readfirstlane(s_count);
      int ns = 0;
      const unsigned long long* sm = sub;
      for (int b = 0; b < kScanBlocks && base_blk + b < nb && count < max_keep; ++b) {
        const int blk = base_blk + b;
        unsigned long long rem = wave_uniform(removed[blk]);
        const int bn = min(64, n - blk * 64);
        const unsigned long long valid = bn >= 64 ? ~0ull : ((1ull << bn) - 1ull);
        // The block's decisions in rounds instead of one box at a time: lane j holds the
        // boxes of the block before j that overlap it (colmask).  A box none of whose
        // overlapping predecessors is still open is settled: removed if one of them is
        // kept, else kept.  The first open box always settles, so at most 64 rounds; boxes
        // suppress few of their neighbours, so a handful.  Same result as the serial pass:
        // a box is settled only when every box that could suppress it has been.
        const unsigned long long before = subcol[b * 64 + lane];
        unsigned long long open = ~rem & valid, keep_bits = 0;
        while (open != 0) {  // wave-uniform
          const bool mine = (open >> lane) & 1ull;
          const bool suppressed = (before & keep_bits) != 0;
          const bool waits = (before & open) != 0;
          const unsigned long long now_removed = __ballot(mine && suppressed);
          const unsigned long long now_kept = __ballot(mine && !suppressed && !waits);
          keep_bits |= now_kept;
          open &= ~(now_kept | now_removed);
        }
        // the serial pass stops at max_keep kept boxes: drop the ones it would not have reached
        for (int extra = __popcll(keep_bits) - (max_keep - count); extra > 0; --extra)
          keep_bits &= ~(1ull << (63 - __builtin_clzll(keep_bits)));
        // the block's kept boxes, in order, written by their own lanes
        if ((keep_bits >> lane) & 1ull) {
          const int pos = __popcll(keep_bits & ((1ull << lane) - 1ull));
          kept[count + pos] = blk * 64 + lane;
          sb_kept[ns + pos] = blk * 64 + lane;
        }
        count += __popcll(keep_bits);
        ns += __popcll(keep_bits);
        // rows kept in this block -> later words of the same super-block
        if (__popcll(keep_bits) > 12) {
          // many: lane (g, w) = (lane / 8, lane % 8) reads word w of rows g, g + 8, ... of the
          // block (the 64 lanes read 512 contiguous bytes at a time), keeps those of kept
          // rows, and the eight row groups are OR-ed across lanes
          const int w8 = lane & 7, g = lane >> 3;
          const unsigned long long* rowp = sm + (b * 64 + g) * kScanBlocks + w8;
          unsigned long long v[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) v[i] = rowp[i * 8 * kScanBlocks];
          unsigned long long acc = 0;
#pragma unroll
          for (int i = 0; i < 8; ++i) acc |= ((keep_bits >> (g + 8 * i)) & 1ull) ? v[i] : 0ull;
#pragma unroll
          for (int o = 8; o < 64; o <<= 1) {
            const unsigned lo = __shfl_xor(static_cast<unsigned>(acc), o, 64);
            const unsigned hi = __shfl_xor(static_cast<unsigned>(acc >> 32), o, 64);
            acc |= (static_cast<unsigned long long>(hi) << 32) | lo;
          }
          if (lane < 8 && w8 > b && base_blk + w8 < nb && acc) removed[base_blk + w8] |= acc;
        } else {
          // few: lane w walks the kept rows, four reads in flight
          const int wl = b + 1 + lane;
          if (wl < kScanBlocks && base_blk + wl < nb) {
            unsigned long long acc = 0, kb = keep_bits;
            const unsigned long long* col = sm + (b * 64) * kScanBlocks + wl;
            while (kb) {
              const int j0 = __builtin_ctzll(kb);
              kb &= kb - 1;
              const int j1 = kb ? __builtin_ctzll(kb) : j0;
              kb &= kb - 1;
              const int j2 = kb ? __builtin_ctzll(kb) : j0;
              kb &= kb - 1;
              const int j3 = kb ? __builtin_ctzll(kb) : j0;
              kb &= kb - 1;
              acc |= (col[j0 * kScanBlocks] | col[j1 * kScanBlocks]) |
                     (col[j2 * kScanBlocks] | col[j3 * kScanBlocks]);
            }
            if (acc) removed[base_blk + wl] |= acc;
          }
        }
        __builtin_amdgcn_wave_barrier();
      }
      if (lane == 0) {
        s_count = count;
        s_ns = ns;
      }
    }
    __syncthreads();
    const int ns = s_ns;
    if (s_count >= max_keep || !more) break;
    // rows kept in this super-block -> words of all later super-blocks
    const int first = base_blk + kScanBlocks, far = nb - first;
    const int total = ns * far;
    for (int p0 = tid; p0 < total; p0 += 4 * kScanThreads) {
      unsigned long long v[4];
      int w[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int p = p0 + u * kScanThreads;
        v[u] = 0;
        w[u] = first;
        if (p < total) {
          const int k = p / far;
          w[u] = first + (p - k * far);
          v[u] = mask[static_cast<long>(sb_kept[k]) * stride + w[u]];
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (v[u]) atomicOr(&removed[w[u]], v[u]);
    }
#pragma unroll
    for (int k = 0; k < kScanLoads; ++k) sub[tid + k * kScanThreads] = ahead[k];
    subcol[tid] = ahead_col;
    __syncthreads();
  }
  if (tid == 0) {
    *num_kept = s_count;
    if (done != nullptr && (final_part || s_count >= max_keep)) *done = 1;
  }
}

// rois[r] = (0, x1, y1, x2, y2) of the r-th kept box (proposal_layer.cpp:187-203).
__global__ void proposal_gather_kernel(const float4* __restrict__ sorted_boxes,
                                       const float* __restrict__ sorted_scores,
                                       const int* __restrict__ kept,
                                       const int* __restrict__ num_kept, float* __restrict__ rois,
                                       float* __restrict__ roi_scores, const int* __restrict__ flags,
                                       int* __restrict__ state, int state_ints) {
  // what the caller learns: state[0] = which equal-score replay ran, state[1] = the result is final
  if (state != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
    state[0] = flags[0];
    if (state_ints > 1) state[1] = 1;
  }
  if (flags[3] != 0) return;  // the head step wrote the rows
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= *num_kept) return;
  const float4 b = sorted_boxes[kept[r]];
  rois[r * 5 + 0] = 0.f;
  rois[r * 5 + 1] = b.x;
  rois[r * 5 + 2] = b.y;
  rois[r * 5 + 3] = b.z;
  rois[r * 5 + 4] = b.w;
  if (roi_scores) roi_scores[r] = sorted_scores[kept[r]];
}

__global__ void zero_ints_kernel(int* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

struct ProposalLayout {
  size_t boxes, scores, k0, v0, k1, v1, korig, kb, vb, seg_lo, seg_hi, pref, posS, posB, mS, mB,
      hole, dest, nseg, cls, sorted_boxes, sorted_scores, mask, kept, flags, total;
};

inline size_t align256(size_t v) { return (v + 255) / 256 * 256; }

ProposalLayout layout(int n, int pre, int post) {
  ProposalLayout L;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    const size_t at = off;
    off += align256(bytes);
    return at;
  };
  const int nb = ceil_div(pre, 64);
  L.boxes = take(sizeof(float4) * n);
  L.scores = take(sizeof(float) * n);
  L.k0 = take(sizeof(uint32_t) * n);
  L.v0 = take(sizeof(int) * n);
  L.k1 = take(sizeof(uint32_t) * n);
  L.v1 = take(sizeof(int) * n);
  L.korig = take(sizeof(uint32_t) * n);
  L.kb = take(sizeof(uint32_t) * n);
  L.vb = take(sizeof(int) * n);
  L.seg_lo = take(sizeof(int) * n);
  L.seg_hi = take(sizeof(int) * n);
  L.pref = take(sizeof(unsigned long long) * n);
  L.posS = take(sizeof(int) * (n + 1));
  L.posB = take(sizeof(int) * (n + 1));
  L.mS = take(sizeof(int) * n);
  L.mB = take(sizeof(int) * n);
  L.hole = take(sizeof(int) * n);
  L.dest = take(sizeof(int) * n);
  L.nseg = take(sizeof(int) * 2 * n);
  L.cls = take(n);
  L.sorted_boxes = take(sizeof(float4) * pre);
  L.sorted_scores = take(sizeof(float) * pre);
  L.mask = take(sizeof(unsigned long long) * (size_t)pre * nb);
  L.kept = take(sizeof(int) * post);
  L.flags = take(sizeof(int) * 8);
  L.total = off;
  return L;
}

}  // namespace
}  // namespace mchip

using namespace mchip;

namespace {

// Scratch of mcProposalStatic: device memory that belongs to the library image, one
// copy per GPU at its own address.  Host code must never pass the array's name to a
// kernel or a copy (on the host it is only a handle for the symbol lookup); the
// per-device address found by static_scratch() is what kernels receive.
constexpr size_t kStaticScratchBytes = size_t(8) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Optional stage timing (measurement hook): while enabled on the calling thread every
// call records up to five HIP events on its stream (a stage that launches nothing shares
// the event before it and reads as zero).
struct ProposalTimes {
  hipEvent_t ev[5];
};
thread_local bool g_prop_timing = false;
thread_local std::vector<ProposalTimes> g_prop_timed;

// Test knob: skip the few-ties replay so that the general one is exercised on every input.
bool g_force_general_replay = false;

constexpr int kMaxDevices = 64;
void* g_scratch_addr[kMaxDevices];
std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch`, looked up once per device.
int static_scratch(void** out) {
  int dev = -1;
  MC_HIP(hipGetDevice(&dev));
  MC_REQUIRE(dev >= 0 && dev < kMaxDevices, "mcProposalStatic: device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_addr[dev]) {
    void* addr = nullptr;
    MC_HIP(hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)));
    MC_REQUIRE(addr != nullptr, "mcProposalStatic: symbol lookup returned no address");
    g_scratch_addr[dev] = addr;
  }
  *out = g_scratch_addr[dev];
  return 0;
}

// Steps of run_proposal: the head of the table alone, the full-size path alone, or both
// (the second then skips itself on the device when the first one settled the result).
constexpr int kStepHead = 1, kStepRest = 2;

// state (device, optional): [0] which equal-score replay ran (0 none, 1 general, 3 few
// ties), [1] 1 when rois / num_rois are final.
int run_proposal(int steps, const float* scores, const float* bbox, const float* im_info,
                 const float* anchors, int A, int H, int W, int feat_stride, float min_size,
                 int pre_nms_topn, int post_nms_topn, float nms_thresh, void* workspace,
                 size_t workspace_bytes, float* rois, float* roi_scores, int* num_rois, int* state,
                 int state_ints, void* stream) {
  MC_REQUIRE(scores && bbox && im_info && anchors && workspace && rois && num_rois,
             "mcProposal: null argument");
  MC_REQUIRE(A > 0 && H > 0 && W > 0 && pre_nms_topn > 0 && post_nms_topn > 0,
             "mcProposal: bad extents");
  const long n_long = (long)A * H * W;
  MC_REQUIRE(n_long < (1L << 24), "mcProposal: too many proposals");
  const int n = static_cast<int>(n_long);
  const int pre = pre_nms_topn < n ? pre_nms_topn : n;
  const ProposalLayout L = layout(n, pre, post_nms_topn);
  MC_REQUIRE(workspace_bytes >= L.total, "mcProposal: workspace too small (%zu < %zu)",
             workspace_bytes, L.total);
  char* ws = static_cast<char*>(workspace);
  float4* boxes = reinterpret_cast<float4*>(ws + L.boxes);
  float* sc = reinterpret_cast<float*>(ws + L.scores);
  uint32_t* k0 = reinterpret_cast<uint32_t*>(ws + L.k0);
  int* v0 = reinterpret_cast<int*>(ws + L.v0);
  uint32_t* k1 = reinterpret_cast<uint32_t*>(ws + L.k1);
  int* v1 = reinterpret_cast<int*>(ws + L.v1);
  uint32_t* korig = reinterpret_cast<uint32_t*>(ws + L.korig);
  auto ints = [&](size_t off) { return reinterpret_cast<int*>(ws + off); };
  float4* sboxes = reinterpret_cast<float4*>(ws + L.sorted_boxes);
  float* sscores = reinterpret_cast<float*>(ws + L.sorted_scores);
  unsigned long long* mask = reinterpret_cast<unsigned long long*>(ws + L.mask);
  int* kept = reinterpret_cast<int*>(ws + L.kept);
  // flags: [0] equal scores among the first pre + 1 sorted places (| 2: the few-ties replay
  // took them), [1] few-ties replay done, [2] the scan settled the result, [3] the head of
  // the table settled it (the full-size path skips itself), [4] entries the head ordered
  int* flags = reinterpret_cast<int*>(ws + L.flags);
  int* done = flags + 2;
  int* complete = flags + 3;
  int* head_info = flags + 4;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int nb = ceil_div(pre, 64);
  // (the equal-score replay's prefix-count array holds the column words of the overlap matrix
  // whenever the replay is not running)
  unsigned long long* colmask = reinterpret_cast<unsigned long long*>(ws + L.pref);

  ProposalTimes times;
  const bool timing = g_prop_timing;
  auto mark = [&](int k) {
    if (!timing) return hipSuccess;
    hipError_t e = hipEventCreate(&times.ev[k]);
    return e != hipSuccess ? e : hipEventRecord(times.ev[k], st);
  };
  MC_HIP(mark(0));
  // foreground scores are the second half of the score blob (proposal_layer.cpp:295)
  proposal_decode_kernel<<<ceil_div(n, 256), 256, 0, st>>>(scores + n, bbox, anchors, im_info, A, H,
                                                          W, feat_stride, min_size, boxes, k0,
                                                          korig, v0, sc, flags);
  MC_LAUNCH_CHECK();
  // The head can settle the result only if post_nms_topn kept boxes fit it (or it is the
  // whole table).
  const bool head_possible = n <= kHeadMaxN && (post_nms_topn < kHeadWant || pre <= kHeadWant);
  if ((steps & kStepHead) && head_possible) {
    const int want = pre < kHeadWant ? pre : kHeadWant, head_nb = ceil_div(want, 64);
    proposal_head_kernel<<<1, kHeadThreads, 0, st>>>(korig, n, want, k1, v1, head_info, boxes, sc,
                                                     sboxes, sscores);
    MC_LAUNCH_CHECK();
    MC_HIP(mark(1));
    nms_mask_kernel<<<head_nb * (head_nb + 1) / 2, 256, 0, st>>>(sboxes, want, nms_thresh, nb, head_nb,
                                                               mask, colmask, nullptr);
    MC_LAUNCH_CHECK();
    nms_scan_kernel<<<1, kScanThreads, sizeof(unsigned long long) * head_nb, st>>>(
        mask, want, head_nb, nb, post_nms_topn, kept, num_rois, done, want == pre, 0, colmask);
    MC_LAUNCH_CHECK();
    proposal_head_check_kernel<<<1, 512, 0, st>>>(k1, head_info, want, kept, num_rois, post_nms_topn,
                                                  mask, nb, flags, sboxes, sscores, rois, roi_scores,
                                                  (steps & kStepRest) ? nullptr : state);
    MC_LAUNCH_CHECK();
  } else {
    MC_HIP(mark(1));
  }
  MC_HIP(mark(2));
  if (steps & kStepRest) {
    if (n <= kSortLdsMax)
      proposal_sort_lds_kernel<<<1, kSortThreads, 0, st>>>(k0, v0, n, pre, flags, complete);
    else
      proposal_sort_kernel<<<1, kSortThreads, 0, st>>>(k0, v0, k1, v1, n, pre, flags, complete);
    MC_LAUNCH_CHECK();
    // both are no-ops unless equal scores reach into the first `pre` places; the first
    // takes inputs with few equal scores, the second everything else
    if (!g_force_general_replay) {
      tie_replay_fast_kernel<<<1, kFastThreads, 0, st>>>(flags, k0, n, pre, reinterpret_cast<uint2*>(ws + L.pref), v0);
      MC_LAUNCH_CHECK();
    }
    quicksort_replay_kernel<<<1, kQsThreads, 0, st>>>(
        flags, korig, n, pre, k1, v1, reinterpret_cast<uint32_t*>(ws + L.kb), ints(L.vb),
        ints(L.seg_lo), ints(L.seg_hi), reinterpret_cast<unsigned long long*>(ws + L.pref),
        ints(L.posS), ints(L.posB), ints(L.mS), ints(L.mB), ints(L.hole), ints(L.dest), ints(L.nseg),
        reinterpret_cast<unsigned char*>(ws + L.cls), v0);
    MC_LAUNCH_CHECK();
    proposal_order_gather_kernel<<<ceil_div(pre, 256), 256, 0, st>>>(v0, pre, boxes, sc, sboxes, sscores,
                                                                     complete);
    MC_LAUNCH_CHECK();
    MC_HIP(mark(3));
    // The greedy pass stops at post_nms_topn kept boxes, usually long before the last
    // candidate: first the best kScanRows candidates among themselves (a corner of the
    // overlap matrix, one super-block of the scan).  If that settles the result the
    // full-size launches behind it return at once; otherwise they fill the whole matrix and
    // the scan resumes behind the first super-block.  (`done` is also set when the head
    // step was complete: all four launches return at once then.)
    const int head = pre < kScanRows ? pre : kScanRows, head_nb = ceil_div(head, 64);
    nms_mask_kernel<<<head_nb * (head_nb + 1) / 2, 256, 0, st>>>(sboxes, head, nms_thresh, nb, head_nb, mask,
                                                               colmask, done);
    MC_LAUNCH_CHECK();
    nms_scan_kernel<<<1, kScanThreads, sizeof(unsigned long long) * head_nb, st>>>(
        mask, head, head_nb, nb, post_nms_topn, kept, num_rois, done, head == pre, 0, colmask);
    MC_LAUNCH_CHECK();
    if (head < pre) {
      nms_mask_kernel<<<std::min(nb * (nb + 1) / 2, 8 * kNumCu), 256, 0, st>>>(sboxes, pre, nms_thresh, nb, nb,
                                                                             mask, colmask, done);
      MC_LAUNCH_CHECK();
      nms_scan_kernel<<<1, kScanThreads, sizeof(unsigned long long) * nb, st>>>(
          mask, pre, nb, nb, post_nms_topn, kept, num_rois, done, 1, 1, colmask);
      MC_LAUNCH_CHECK();
    }
    proposal_gather_kernel<<<ceil_div(post_nms_topn, 256), 256, 0, st>>>(
        sboxes, sscores, kept, num_rois, rois, roi_scores, flags, state, state_ints);
    MC_LAUNCH_CHECK();
  } else {
    times.ev[3] = times.ev[2];  // (nothing ran in stage 2: no event of its own, zero time)
    if (state && !head_possible) {  // the head step was asked for and cannot run: not final
      zero_ints_kernel<<<1, 64, 0, st>>>(state, state_ints);
      MC_LAUNCH_CHECK();
      MC_HIP(mark(4));
    } else {
      times.ev[4] = times.ev[3];
    }
  }
  if (steps & kStepRest) MC_HIP(mark(4));
  if (timing) g_prop_timed.push_back(times);
  return 0;
}


}  // namespace

extern "C" {

int mcProposalWorkspaceSize(int num_proposals, int pre_nms_topn, int post_nms_topn,
                            size_t* bytes) {
  MC_REQUIRE(bytes && num_proposals > 0 && pre_nms_topn > 0 && post_nms_topn > 0,
             "mcProposalWorkspaceSize: bad argument");
  const int pre = pre_nms_topn < num_proposals ? pre_nms_topn : num_proposals;
  *bytes = layout(num_proposals, pre, post_nms_topn).total;
  return 0;
}

int mcProposal(const float* scores, const float* bbox, const float* im_info, const float* anchors,
               int A, int H, int W, int feat_stride, float min_size, int pre_nms_topn,
               int post_nms_topn, float nms_thresh, void* workspace, size_t workspace_bytes,
               float* rois, float* roi_scores, int* num_rois, int* tie_flag, void* stream) {
  return run_proposal(kStepHead | kStepRest, scores, bbox, im_info, anchors, A, H, W, feat_stride,
                      min_size, pre_nms_topn, post_nms_topn, nms_thresh, workspace, workspace_bytes,
                      rois, roi_scores, num_rois, tie_flag, 1, stream);
}

int mcProposalHead(const float* scores, const float* bbox, const float* im_info, const float* anchors,
                   int A, int H, int W, int feat_stride, float min_size, int pre_nms_topn,
                   int post_nms_topn, float nms_thresh, void* workspace, size_t workspace_bytes,
                   float* rois, float* roi_scores, int* num_rois, int* state, void* stream) {
  MC_REQUIRE(state, "mcProposalHead: null argument");
  return run_proposal(kStepHead, scores, bbox, im_info, anchors, A, H, W, feat_stride, min_size,
                      pre_nms_topn, post_nms_topn, nms_thresh, workspace, workspace_bytes, rois,
                      roi_scores, num_rois, state, 2, stream);
}

int mcProposalRest(const float* scores, const float* bbox, const float* im_info, const float* anchors,
                   int A, int H, int W, int feat_stride, float min_size, int pre_nms_topn,
                   int post_nms_topn, float nms_thresh, void* workspace, size_t workspace_bytes,
                   float* rois, float* roi_scores, int* num_rois, int* state, void* stream) {
  return run_proposal(kStepRest, scores, bbox, im_info, anchors, A, H, W, feat_stride, min_size,
                      pre_nms_topn, post_nms_topn, nms_thresh, workspace, workspace_bytes, rois,
                      roi_scores, num_rois, state, 2, stream);
}

int mcProposalForceGeneralReplay(int on) {
  g_force_general_replay = on != 0;
  return 0;
}

int mcProposalTimingEnable(int on) {
  g_prop_timing = on != 0;
  return 0;
}

int mcProposalTimingCollect(double* stage_ms, long* calls) {
  double sum[4] = {0., 0., 0., 0.};
  for (auto& t : g_prop_timed) {
    MC_HIP(hipEventSynchronize(t.ev[4]));
    for (int k = 0; k < 4; ++k) {
      float e = 0.f;
      MC_HIP(hipEventElapsedTime(&e, t.ev[k], t.ev[k + 1]));
      sum[k] += e;
    }
    for (int k = 0; k < 5; ++k)
      if (k == 0 || t.ev[k] != t.ev[k - 1]) (void)hipEventDestroy(t.ev[k]);  // (an empty stage shares its event)
  }
  if (stage_ms)
    for (int k = 0; k < 4; ++k) stage_ms[k] = sum[k];
  if (calls) *calls = static_cast<long>(g_prop_timed.size());
  g_prop_timed.clear();
  return 0;
}

int mcProposalStatic(const float* scores, const float* bbox, const float* im_info,
                     const float* anchors, int A, int H, int W, int feat_stride, float min_size,
                     int pre_nms_topn, int post_nms_topn, float nms_thresh, float* rois,
                     float* roi_scores, int* num_rois, int* tie_flag, void* stream) {
  MC_REQUIRE(A > 0 && H > 0 && W > 0 && pre_nms_topn > 0 && post_nms_topn > 0,
             "mcProposalStatic: bad extents");
  const long n_long = (long)A * H * W;
  MC_REQUIRE(n_long < (1L << 24), "mcProposalStatic: too many proposals");
  const int n = static_cast<int>(n_long);
  const size_t need = layout(n, pre_nms_topn < n ? pre_nms_topn : n, post_nms_topn).total;
  MC_REQUIRE(need <= kStaticScratchBytes,
             "mcProposalStatic: this problem needs %zu bytes of scratch, the built-in buffer holds "
             "%zu; use mcProposal with a caller-owned workspace",
             need, kStaticScratchBytes);
  void* ws = nullptr;
  if (static_scratch(&ws) != 0) return -1;
  return run_proposal(kStepHead | kStepRest, scores, bbox, im_info, anchors, A, H, W, feat_stride,
                      min_size, pre_nms_topn, post_nms_topn, nms_thresh, ws, kStaticScratchBytes, rois,
                      roi_scores, num_rois, tie_flag, 1, stream);
}

}  // extern "C"
