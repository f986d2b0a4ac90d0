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
__device__ __forceinline__ uint32_t desc_key(float f) {
  uint32_t u = __float_as_uint(f);
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
__device__ inline void block_sort_desc_lds(uint32_t* keys, VT* vals, int n, BlockSortLds16* lds) {
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

}  // namespace mchip

#endif  // MCHIP_EXACT_BLOCK_SORT_H_
