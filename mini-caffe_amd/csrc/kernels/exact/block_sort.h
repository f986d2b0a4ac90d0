// Stable descending sort of float keys by one 512-thread workgroup.
//
// LSD radix sort, 4 bits per pass, 8 passes.  Every thread owns a contiguous
// run of the input and a private column of the digit histogram, so ranks follow
// (thread, position) order and equal keys keep their input order: the result is
// ordered by (key descending, original position ascending), which is what
// std::stable_sort with a "greater" comparator produces on the host.
#ifndef MCHIP_EXACT_BLOCK_SORT_H_
#define MCHIP_EXACT_BLOCK_SORT_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mchip {

constexpr int kSortThreads = 512;

// Monotone map float -> uint32 such that a > b  <=>  key(a) < key(b); -0 == +0.
__host__ __device__ __forceinline__ uint32_t desc_key(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if (u == 0x80000000u) u = 0u;
  const uint32_t asc = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return ~asc;
}

struct BlockSortLds {
  uint32_t counts[16 * kSortThreads];
  uint32_t wave_sum[kSortThreads / 64];
};

// Exclusive prefix sum of one value per thread over the workgroup.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* wave_sum) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const uint32_t u = __shfl_up(inc, o, 64);
    if (lane >= o) inc += u;
  }
  __syncthreads();
  if (lane == 63) wave_sum[wave] = inc;
  __syncthreads();
  uint32_t base = 0;
  for (int w = 0; w < wave; ++w) base += wave_sum[w];
  return base + inc - v;
}

// Sorts (k0, v0)[0..n) into descending key order.  k0/v0 and k1/v1 are two
// global scratch pairs of n entries; the result ends up in k0/v0 (8 passes).
// All threads of the workgroup must call it.
__device__ inline void block_sort_desc(uint32_t* k0, int* v0, uint32_t* k1, int* v1, int n,
                                       BlockSortLds* lds) {
  const int tid = threadIdx.x;
  const int per = (n + kSortThreads - 1) / kSortThreads;
  const int begin = min(tid * per, n), end = min(begin + per, n);
  uint32_t* kin = k0;
  int* vin = v0;
  uint32_t* kout = k1;
  int* vout = v1;
  for (int shift = 0; shift < 32; shift += 4) {
#pragma unroll
    for (int d = 0; d < 16; ++d) lds->counts[d * kSortThreads + tid] = 0;
    for (int i = begin; i < end; ++i) lds->counts[((kin[i] >> shift) & 15u) * kSortThreads + tid]++;
    __syncthreads();
    // flattened [digit][thread] order == final rank order; thread t scans 16 entries
    uint32_t local[16], sum = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      local[j] = lds->counts[tid * 16 + j];
      sum += local[j];
    }
    uint32_t run = block_exclusive_scan(sum, lds->wave_sum);
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      lds->counts[tid * 16 + j] = run;
      run += local[j];
    }
    __syncthreads();
    for (int i = begin; i < end; ++i) {
      const uint32_t k = kin[i];
      const uint32_t pos = lds->counts[((k >> shift) & 15u) * kSortThreads + tid]++;
      kout[pos] = k;
      vout[pos] = vin[i];
    }
    __syncthreads();
    __threadfence_block();
    uint32_t* tk = kin; kin = kout; kout = tk;
    int* tv = vin; vin = vout; vout = tv;
  }
}

// The same sort with keys and values resident in LDS and sorted in place: per
// pass every thread takes its contiguous run into registers, counts digits in
// its private histogram column, the workgroup synchronises, and each thread
// scatters its run back.  16-bit histogram entries and ranks: n < 65536.
// MAXPER bounds the run length: n <= MAXPER * kSortThreads.  VT is the value
// type (unsigned short halves the LDS footprint when values are indices < 65536).
struct BlockSortLds16 {
  unsigned short counts[16 * kSortThreads];
  uint32_t wave_sum[kSortThreads / 64];
};

template <int MAXPER, typename VT, bool SKIP_CONSTANT_DIGITS = true>
__device__ __forceinline__ void block_sort_desc_lds(uint32_t* keys, VT* vals, int n, BlockSortLds16* lds) {
  const int tid = threadIdx.x;
  const int per = (n + kSortThreads - 1) / kSortThreads;
  const int begin = min(tid * per, n), end = min(begin + per, n);
  const int cnt = end - begin;
  // Bits in which any two keys differ: a pass over a digit that is the same in every
  // key is the identity (the sort is stable) and is skipped.  Softmax scores over many
  // classes share their sign and most of their exponent, which saves two of the 8
  // passes; callers whose keys spread over all exponents switch the look-ahead off.
  uint32_t diff = 0xffffffffu;
  if constexpr (SKIP_CONSTANT_DIGITS) {
    diff = 0;
    const uint32_t first = n > 0 ? keys[0] : 0u;
    for (int j = 0; j < cnt; ++j) diff |= keys[begin + j] ^ first;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) diff |= __shfl_xor(diff, o, 64);
    if ((tid & 63) == 0) lds->wave_sum[tid >> 6] = diff;
    __syncthreads();
    diff = 0;
#pragma unroll
    for (int w = 0; w < kSortThreads / 64; ++w) diff |= lds->wave_sum[w];
    __syncthreads();  // wave_sum is used again by the scans below
  }
  for (int shift = 0; shift < 32; shift += 4) {
    if (((diff >> shift) & 15u) == 0u) continue;  // uniform over the workgroup
    uint32_t rk[MAXPER];
    VT rv[MAXPER];
#pragma unroll
    for (int j = 0; j < MAXPER; ++j)
      if (j < cnt) {
        rk[j] = keys[begin + j];
        rv[j] = vals[begin + j];
      }
#pragma unroll
    for (int d = 0; d < 16; ++d) lds->counts[d * kSortThreads + tid] = 0;
#pragma unroll
    for (int j = 0; j < MAXPER; ++j)
      if (j < cnt) lds->counts[((rk[j] >> shift) & 15u) * kSortThreads + tid]++;
    __syncthreads();
    // flattened [digit][thread] order == final rank order; thread t scans 16 entries
    uint32_t local[16], sum = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      local[j] = lds->counts[tid * 16 + j];
      sum += local[j];
    }
    uint32_t run = block_exclusive_scan(sum, lds->wave_sum);
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      lds->counts[tid * 16 + j] = static_cast<unsigned short>(run);
      run += local[j];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < MAXPER; ++j)
      if (j < cnt) {
        const uint32_t pos = lds->counts[((rk[j] >> shift) & 15u) * kSortThreads + tid]++;
        keys[pos] = rk[j];
        vals[pos] = rv[j];
      }
    __syncthreads();
  }
}

// ---- the `want` smallest keys of a table, in order, without sorting the table --------
//
// For want <= kSortThreads (the candidates of a greedy pass that looks at a few hundred
// entries of a table of thousands).  Every thread holds PER keys in registers, entry
// tid + j * kSortThreads in rk[j]; the all-ones key marks "no entry".
//   1. First cut: every thread has a smallest key; in each wavefront the ceil(want / 8)-th
//      smallest of those has that many keys at or below it, so the largest of the eight
//      wavefronts' values has at least `want`.  The threads hold strided samples of the
//      table, so usually a thousand or two keys pass: the candidates (kSelectCandPer per
//      thread at most, else the call fails and the caller sorts).
//      If they fit one to a thread they all go through step 3 and step 2 is skipped.
//   2. tau = the want-th smallest candidate by bisection on the key bits, two bits per
//      round from the top (three trial values, one count over the workgroup each: ballots
//      and scalar population counts within a wavefront, the wavefronts' counts through
//      LDS); bits that are the same in every candidate are skipped.
//   3. The m >= want candidates at or below tau (more than want only if keys equal to tau
//      hang over) go one to a thread through a compare-exchange network on (key, index):
//      all pairs differ, so the order is that of a stable sort by key.
// Returns m, and in thread t < m the entry of rank t; 0 when step 1 or 3 does not fit
// (crowds of equal keys).  All threads of the workgroup must call it.  A caller that already
// knows a key with at least `want` entries at or below it passes it as `known_cut` (not 0)
// and step 1 uses that instead of the thread minima.
constexpr int kSelectCandPer = 8;
struct BlockSelectLds {
  uint32_t ckey[kSelectCandPer * kSortThreads];
  unsigned short cidx[kSelectCandPer * kSortThreads];
  uint32_t x[2 * kSortThreads];
  int cnt[2][3][kSortThreads / 64];
  uint32_t red[kSortThreads / 64];
  uint32_t wave_sum[kSortThreads / 64];
  int tot;
};

template <int K, int J>
__device__ __forceinline__ void bitonic_step(uint32_t& key, uint32_t& idx, uint32_t* xk, uint32_t* xi) {
  const int tid = threadIdx.x;
  uint32_t ok, oi;
  if constexpr (J >= 64) {
    __syncthreads();
    xk[tid] = key;
    xi[tid] = idx;
    __syncthreads();
    ok = xk[tid ^ J];
    oi = xi[tid ^ J];
  } else {
    ok = __shfl_xor(key, J, 64);
    oi = __shfl_xor(idx, J, 64);
  }
  const bool up = (tid & K) == 0;          // this run sorts ascending
  const bool lower = (tid & J) == 0;       // this thread keeps the smaller of the two
  const bool other_less = ok < key || (ok == key && oi < idx);
  const bool take = (lower == up) ? other_less : !other_less;
  key = take ? ok : key;
  idx = take ? oi : idx;
  if constexpr (J > 1) bitonic_step<K, J / 2>(key, idx, xk, xi);
}
// Ascending by (key, idx) over one pair per thread of a kSortThreads workgroup; fully
// unrolled, so every lane shuffle has a constant distance.
template <int K>
__device__ __forceinline__ void bitonic_sort_block(uint32_t& key, uint32_t& idx, uint32_t* xk, uint32_t* xi) {
  if constexpr (K > 2) bitonic_sort_block<K / 2>(key, idx, xk, xi);
  bitonic_step<K, K / 2>(key, idx, xk, xi);
}

template <int PER>
__device__ __forceinline__ int block_select_smallest(const uint32_t (&rk)[PER], int want, BlockSelectLds* s,
                                            uint32_t* key_out, uint32_t* idx_out, uint32_t known_cut = 0) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t lowest = 0xffffffffu;
#pragma unroll
  for (int j = 0; j < PER; ++j) lowest = min(lowest, rk[j]);
  if (known_cut != 0) lowest = known_cut;  // (uniform) the caller knows a key with `want` entries at or below it
  // the wavefront's share of the cut: the ceil(want / 8)-th smallest of its 64 thread
  // minima (eight wavefronts: at least `want` entries lie at or below the largest share)
  uint32_t cut = lowest;  // (a thread without entries holds all ones)
  static_assert(kSortThreads / 64 == 8, "eight wavefronts share the cut");
  const int kth = (want + 7) / 8;
  if (kth >= 64 || known_cut != 0) {  // uniform: the largest of the 64 (all the same with a known cut)
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cut = max(cut, static_cast<uint32_t>(__shfl_xor(cut, o, 64)));
  } else {  // the 64 minima in ascending order over the lanes, then the kth of them
#pragma unroll
    for (int k = 2; k <= 64; k <<= 1) {
#pragma unroll
      for (int j = k >> 1; j > 0; j >>= 1) {
        const uint32_t other = static_cast<uint32_t>(__shfl_xor(cut, j, 64));
        const bool up = (lane & k) == 0 || k == 64, lower = (lane & j) == 0;
        cut = (lower == up) ? min(cut, other) : max(cut, other);
      }
    }
    cut = static_cast<uint32_t>(__shfl(cut, kth - 1, 64));
  }
  __syncthreads();  // (the caller may still be reading what `s` overlays)
  if (lane == 0) s->red[wave] = cut;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kSortThreads / 64; ++w) cut = max(cut, s->red[w]);
  int mine = 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) mine += (rk[j] != 0xffffffffu && rk[j] <= cut) ? 1 : 0;
  uint32_t base = block_exclusive_scan(static_cast<uint32_t>(mine), s->wave_sum);
  if (tid == kSortThreads - 1) s->tot = static_cast<int>(base) + mine;
  __syncthreads();
  const int ncand = s->tot;
  if (ncand > kSelectCandPer * kSortThreads || ncand < want) return 0;  // uniform
  {
    int at = static_cast<int>(base);
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (rk[j] != 0xffffffffu && rk[j] <= cut) {
        s->ckey[at] = rk[j];
        s->cidx[at] = static_cast<unsigned short>(tid + j * kSortThreads);
        ++at;
      }
  }
  __syncthreads();
  if (ncand <= kSortThreads) {  // uniform
    // the candidates fit one to a thread: order them all; m = those at or below the
    // want-th of them
    uint32_t key = tid < ncand ? s->ckey[tid] : 0xffffffffu;
    uint32_t idx = tid < ncand ? s->cidx[tid] : 0xffffffffu;
    bitonic_sort_block<kSortThreads>(key, idx, s->x, s->x + kSortThreads);
    __syncthreads();
    if (tid == want - 1) s->x[0] = key;
    __syncthreads();
    const uint32_t tau = s->x[0];
    *key_out = key;
    *idx_out = idx;
    return __syncthreads_count(tid < ncand && key <= tau);
  }
  uint32_t ck[kSelectCandPer];
  uint32_t diff = 0;
  const uint32_t first = s->ckey[0];
#pragma unroll
  for (int j = 0; j < kSelectCandPer; ++j) {
    const int i = tid + j * kSortThreads;
    ck[j] = i < ncand ? s->ckey[i] : 0xffffffffu;
    diff |= (i < ncand ? ck[j] : first) ^ first;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) diff |= __shfl_xor(diff, o, 64);
  if (lane == 0) s->red[wave] = diff;  // (all reads of the cut are behind two barriers)
  __syncthreads();
  diff = 0;
#pragma unroll
  for (int w = 0; w < kSortThreads / 64; ++w) diff |= s->red[w];
  diff = __builtin_amdgcn_readfirstlane(diff);
  // Of the four values of a bit pair the smallest whose trial (prefix | pair | all lower
  // bits set) has enough candidates at or below.  (An absent entry, all ones, is never at
  // or below a trial value that has a zero bit; the all-ones trial is not counted.)
  uint32_t tau = first & ~diff;
  for (int bit = 31; bit >= 1; bit -= 2) {
    if (!((diff >> (bit - 1)) & 3u)) continue;  // uniform
    const uint32_t pair = 3u << (bit - 1), low = (1u << (bit - 1)) - 1u;
    const uint32_t prefix = tau & ~pair;
    const uint32_t t0 = prefix | low, t1 = prefix | (1u << (bit - 1)) | low, t2 = prefix | (1u << bit) | low;
    int c0 = 0, c1 = 0, c2 = 0;
#pragma unroll
    for (int j = 0; j < kSelectCandPer; ++j) {
      c0 += __popcll(__ballot(ck[j] <= t0));  // scalar: the wavefront's count
      c1 += __popcll(__ballot(ck[j] <= t1));
      c2 += __popcll(__ballot(ck[j] <= t2));
    }
    const int slot = (bit >> 1) & 1;
    if (lane == 0) {
      s->cnt[slot][0][wave] = c0;
      s->cnt[slot][1][wave] = c1;
      s->cnt[slot][2][wave] = c2;
    }
    __syncthreads();
    int n0 = 0, n1 = 0, n2 = 0;
#pragma unroll
    for (int w = 0; w < kSortThreads / 64; ++w) {
      n0 += s->cnt[slot][0][w];
      n1 += s->cnt[slot][1][w];
      n2 += s->cnt[slot][2][w];
    }
    tau = prefix | (n0 >= want ? 0u : n1 >= want ? (1u << (bit - 1)) : n2 >= want ? (1u << bit) : pair);
  }
  mine = 0;
#pragma unroll
  for (int j = 0; j < kSelectCandPer; ++j) mine += (ck[j] != 0xffffffffu && ck[j] <= tau) ? 1 : 0;
  base = block_exclusive_scan(static_cast<uint32_t>(mine), s->wave_sum);
  if (tid == kSortThreads - 1) s->tot = static_cast<int>(base) + mine;
  __syncthreads();
  const int m = s->tot;
  if (m > kSortThreads) return 0;  // uniform: keys equal to tau in a crowd
  {
    int at = static_cast<int>(base);
#pragma unroll
    for (int j = 0; j < kSelectCandPer; ++j)
      if (ck[j] != 0xffffffffu && ck[j] <= tau) {
        s->x[at] = ck[j];
        s->x[kSortThreads + at] = s->cidx[tid + j * kSortThreads];
        ++at;
      }
  }
  __syncthreads();
  uint32_t key = tid < m ? s->x[tid] : 0xffffffffu;
  uint32_t idx = tid < m ? s->x[kSortThreads + tid] : 0xffffffffu;
  bitonic_sort_block<kSortThreads>(key, idx, s->x, s->x + kSortThreads);
  *key_out = key;
  *idx_out = idx;
  return m;
}

}  // namespace mchip

#endif  // MCHIP_EXACT_BLOCK_SORT_H_
