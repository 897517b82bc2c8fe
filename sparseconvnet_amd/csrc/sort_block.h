// The sort of a few thousand (64-bit key, 32-bit value) pairs by one workgroup of 1024 threads,
// as a device function: k_rs_single (sort.hip) is this and nothing else, and the rulebook kernels of
// the smallest levels (metadata.hip) sort their tap patterns with it without leaving the kernel.
// The deep levels of a network are a few hundred to a few thousand sites, and what their rulebooks
// cost is launches.
#pragma once
#include <hip/hip_runtime.h>

namespace scn {

typedef unsigned long long u64;

// Rank of each of a wavefront's ITEMS x 64 pairs (round r, lane) among the pairs of its quarter
// with the same digit value, in round-major order; cnt[0 .. 2^bits) (this wavefront's, zero on entry)
// ends as the quarter's count of every value.
template <int ITEMS>
__device__ inline void rank_quarter(const unsigned (&digit)[ITEMS], const bool (&valid)[ITEMS], int bits, int *cnt,
                                    int lane, int (&rank)[ITEMS]) {
  const u64 below = (1ull << lane) - 1ull;
#pragma unroll
  for (int r = 0; r < ITEMS; r++) {
    u64 peers = __ballot(valid[r]);
    if (!peers) {  // a round past the end of the input (the whole wavefront agrees)
      rank[r] = 0;
      continue;
    }
    for (int b = 0; b < bits; b++) {
      const u64 has = __ballot((digit[r] >> b) & 1u);
      peers &= ((digit[r] >> b) & 1u) ? has : ~has;
    }
    const int before = __popcll(peers & below);
    int old = 0;
    if (valid[r]) old = cnt[digit[r]];  // every lane of the group reads the count before its first lane bumps it
    if (valid[r] && before == 0) cnt[digit[r]] = old + __popcll(peers);
    rank[r] = old + before;
  }
}

// Sixteen wavefronts each keep a contiguous ITEMS x 64 pairs in registers (pair i of the input:
// wavefront i / (64 ITEMS), round (i / 64) % ITEMS, lane i % 64) and rank them as the tiled scatter
// kernel does, with digits of `width` <= 8 bits (the prefix over 16 wavefronts' counts of every digit
// value is what a pass costs here, so fewer values beat fewer passes); the pairs change places
// through LDS between digits.  Stable.  Every thread of the workgroup calls it; on return
// sh.skey / sh.sval hold the sorted pairs (a barrier has been passed).
constexpr int RS1_THREADS = 1024, RS1_WAVES = 16;
constexpr int RS1_BITS = 8, RS1_BINS = 1 << RS1_BITS;
template <int ITEMS> struct BlockSort {
  int cnt[RS1_WAVES][RS1_BINS];
  int lstart[RS1_BINS];
  int wsum[RS1_BINS / 64];
  u64 skey[RS1_THREADS * ITEMS];
  int sval[RS1_THREADS * ITEMS];
};
template <int ITEMS>
__device__ inline void block_sort(BlockSort<ITEMS> &sh, u64 (&key)[ITEMS], int (&val)[ITEMS], const bool (&valid)[ITEMS],
                                  int end_bit, int width) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int q0 = wave * (ITEMS * 64);
  unsigned digit[ITEMS];
  int rank[ITEMS];
  for (int shift = 0; shift < end_bit; shift += width) {
    const int bits = min(width, end_bit - shift), bins = 1 << bits;
    const unsigned mask = (unsigned)bins - 1u;
    for (int e = threadIdx.x; e < RS1_WAVES * bins; e += RS1_THREADS) sh.cnt[e / bins][e % bins] = 0;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < ITEMS; r++) digit[r] = (unsigned)(key[r] >> shift) & mask;
    rank_quarter<ITEMS>(digit, valid, bits, sh.cnt[wave], lane, rank);
    __syncthreads();
    // thread d < bins: the counts of value d become their exclusive prefix over the wavefronts;
    // then an exclusive scan of the totals over d (the first bins / 64 wavefronts)
    int total = 0;
    if (threadIdx.x < bins) {
      for (int w = 0; w < RS1_WAVES; w++) {
        const int c = sh.cnt[w][threadIdx.x];
        sh.cnt[w][threadIdx.x] = total;
        total += c;
      }
    }
    int incl = total;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    if (lane == 63 && wave < RS1_BINS / 64) sh.wsum[wave] = incl;
    __syncthreads();
    if (threadIdx.x < bins) {
      int run = incl - total;
      for (int w = 0; w < wave; w++) run += sh.wsum[w];
      sh.lstart[threadIdx.x] = run;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
      if (!valid[r]) continue;
      const int at = sh.lstart[digit[r]] + sh.cnt[wave][digit[r]] + rank[r];
      sh.skey[at] = key[r];
      sh.sval[at] = val[r];
    }
    __syncthreads();
    if (shift + width < end_bit) {  // the pairs of this wavefront's range for the next digit
#pragma unroll
      for (int r = 0; r < ITEMS; r++) {
        const int i = q0 + r * 64 + lane;
        key[r] = valid[r] ? sh.skey[i] : 0ull;
        val[r] = valid[r] ? sh.sval[i] : 0;
      }
      __syncthreads();
    }
  }
}

}  // namespace scn
