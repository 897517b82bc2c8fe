// Stable least-significant-digit radix sort of (64-bit key, 32-bit value) pairs by the low
// `end_bit` bits of the key: what the rulebook builders sort by (site keys of an input layer,
// candidate output sites of a strided rulebook, tap patterns of a neighbour table).  These are
// tens of thousands to a few million pairs with 16 to 48 significant key bits: small enough
// that a general-purpose library sort spends its time in launches (a histogram pass, then per
// digit a look-back scan with two state fills in front), which is what this file avoids.
//
// Per digit (up to 10 bits) three launches, none of which waits on another workgroup:
//   k_rs_hist     per tile of TILE pairs, the count of every digit value   hist[digit][tile]
//   k_rs_colscan  per digit value, the exclusive prefix over tiles (in place) and the total
//   k_rs_scatter  per tile: rank every pair among the tile's pairs of the same digit value
//                 (stable), add the tile's prefix and the digit value's base (exclusive scan of
//                 the totals, recomputed by every workgroup), write the pair there.
// Ranking inside a tile: wavefront w owns a contiguous quarter of the tile and walks it 64 pairs
// at a time; the lanes of a round that hold the same digit value find each other with one
// ballot per digit bit, the first of them reads and bumps the wavefront's running count of that value in LDS
// (only this wavefront touches its counts, so no barrier), which gives every pair its rank
// inside the wavefront's quarter; a prefix over the four wavefronts' counts then orders the
// quarters.  (Between four and thirty-two thousand pairs the library's merge sort is faster and the
// callers use it; up to 4096 pairs k_rs_single sorts in one launch, see there.)
// The input arrays are not written: passes alternate between the output arrays and scratch.
// The number of pairs may live on the device only (n_dev): the launches are then sized for an
// upper bound and tiles past the real end find nothing to do.
#include "metadata.h"
#include "sort_block.h"

namespace scn {

constexpr int RS_THREADS = 256, RS_WAVES = 4;  // a tile is RS_THREADS * ITEMS pairs: 4096 (large inputs) down to 512
constexpr int RS_MAX_BITS = 10, RS_MAX_BINS = 1 << RS_MAX_BITS;  // widest digit of the tiled kernels (measured on a million
// pairs of 35 bits: four digits of 9 bits beat three of 11 and five of 7; 40 bits sort in four digits of 10)

// The tile's digit counts.  Four times the scatter kernel's threads per tile (the same tiles): the
// kernel is a read of the keys and a few LDS atomics per thread, and one 256-thread workgroup per
// compute unit leaves most of the memory system idle (a million pairs: 9.3 -> 5 us per pass).
template <int RS_ITEMS>
__global__ __launch_bounds__(RS_THREADS *(RS_ITEMS >= 4 ? 4 : RS_ITEMS)) void k_rs_hist(
    const u64 *__restrict__ keys, int64_t n, int shift, int bits, int tiles, int *__restrict__ hist,
    const int *__restrict__ n_dev) {
  constexpr int THREADS = RS_THREADS * (RS_ITEMS >= 4 ? 4 : RS_ITEMS), PER = RS_THREADS * RS_ITEMS / THREADS;
  __shared__ int h[RS_MAX_BINS];
  if (n_dev) n = *n_dev;  // the number of pairs when only the device knows it (n: an upper bound the grid was sized for)
  const int bins = 1 << bits;
  for (int d = threadIdx.x; d < bins; d += THREADS) h[d] = 0;
  __syncthreads();
  const unsigned mask = (unsigned)bins - 1u;
  constexpr int RS_TILE = RS_THREADS * RS_ITEMS;
  const int64_t base = (int64_t)blockIdx.x * RS_TILE;
#pragma unroll
  for (int r = 0; r < PER; r++) {
    const int64_t i = base + r * THREADS + threadIdx.x;
    if (i < n) atomicAdd(&h[(unsigned)(keys[i] >> shift) & mask], 1);
  }
  __syncthreads();
  for (int d = threadIdx.x; d < bins; d += THREADS) hist[(size_t)d * tiles + blockIdx.x] = h[d];
}

// One workgroup (64 threads) per digit value: hist[d][*] becomes its exclusive prefix over tiles,
// tot[d] the sum.
__global__ __launch_bounds__(64) void k_rs_colscan(int *__restrict__ hist, int tiles, int *__restrict__ tot) {
  int *col = hist + (size_t)blockIdx.x * tiles;
  const int lane = threadIdx.x;
  const int per = (tiles + 63) / 64;
  const int t0 = min(tiles, lane * per), t1 = min(tiles, t0 + per);
  int sum = 0;
  for (int t = t0; t < t1; t++) sum += col[t];
  int incl = sum;  // inclusive scan over the 64 lanes
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  int run = incl - sum;
  for (int t = t0; t < t1; t++) {
    const int c = col[t];
    col[t] = run;
    run += c;
  }
  if (lane == 63) tot[blockIdx.x] = incl;
}

template <int RS_ITEMS>
__global__ __launch_bounds__(RS_THREADS) void k_rs_scatter(const u64 *__restrict__ kin, const int *__restrict__ vin,
                                                           u64 *__restrict__ kout, int *__restrict__ vout, int64_t n,
                                                           int shift, int bits, int tiles, const int *__restrict__ offs,
                                                           const int *__restrict__ tot, const int *__restrict__ n_dev) {
  constexpr int RS_TILE = RS_THREADS * RS_ITEMS;
  if (n_dev) n = *n_dev;
  __shared__ int cnt[RS_WAVES][RS_MAX_BINS];
  __shared__ int base[RS_MAX_BINS];    // where the tile's first pair of each digit value goes
  __shared__ int lstart[RS_MAX_BINS];  // the same inside the tile: pairs of smaller digit values
  __shared__ int wsum[RS_WAVES], wsum2[RS_WAVES];
  __shared__ u64 skey[RS_TILE];        // the tile's pairs in the order they leave in
  __shared__ int sval[RS_TILE];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int bins = 1 << bits;
  const unsigned mask = (unsigned)bins - 1u;
  const int per = (bins + RS_THREADS - 1) / RS_THREADS;  // digit values per thread, 1 to 4
  const int d0 = threadIdx.x * per;
  // exclusive scan of the digit values' totals (thread t: values [t * per, (t + 1) * per)) + this tile's prefix
  {
    int mine = 0;
    for (int j = 0; j < per; j++)
      if (d0 + j < bins) mine += tot[d0 + j];
    int incl = mine;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    if (lane == 63) wsum[wave] = incl;
    for (int d = threadIdx.x; d < bins; d += RS_THREADS) {
#pragma unroll
      for (int w = 0; w < RS_WAVES; w++) cnt[w][d] = 0;
    }
    __syncthreads();
    int run = incl - mine;
    for (int w = 0; w < wave; w++) run += wsum[w];
    for (int j = 0; j < per; j++)
      if (d0 + j < bins) {
        base[d0 + j] = run + offs[(size_t)(d0 + j) * tiles + blockIdx.x];
        run += tot[d0 + j];
      }
  }
  // this wavefront's quarter: pairs [q0, q0 + ITEMS * 64)
  const int64_t q0 = (int64_t)blockIdx.x * RS_TILE + (int64_t)wave * (RS_ITEMS * 64);
  u64 key[RS_ITEMS];
  int val[RS_ITEMS];
  unsigned digit[RS_ITEMS];
  bool valid[RS_ITEMS];
  int rank[RS_ITEMS];
#pragma unroll
  for (int r = 0; r < RS_ITEMS; r++) {
    const int64_t i = q0 + r * 64 + lane;
    valid[r] = i < n;
    key[r] = valid[r] ? kin[i] : 0ull;
    val[r] = valid[r] ? vin[i] : 0;
    digit[r] = (unsigned)(key[r] >> shift) & mask;
  }
  rank_quarter<RS_ITEMS>(digit, valid, bits, cnt[wave], lane, rank);
  __syncthreads();  // all four quarters counted, base[] written
  // The tile's own exclusive prefix over digit values: a pair leaves the tile at lstart[d] + (pairs
  // of the same value before it), so that what goes to consecutive addresses of the output sits
  // at consecutive places of the tile and is written by consecutive lanes (a lane writing its own
  // pair where it belongs touched one 32-byte sector per 8- or 4-byte store).
  {
    int mine = 0;
    for (int j = 0; j < per; j++)
      if (d0 + j < bins)
        for (int w = 0; w < RS_WAVES; w++) mine += cnt[w][d0 + j];
    int incl = mine;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    if (lane == 63) wsum2[wave] = incl;
    __syncthreads();
    int run = incl - mine;
    for (int w = 0; w < wave; w++) run += wsum2[w];
    for (int j = 0; j < per; j++)
      if (d0 + j < bins) {
        lstart[d0 + j] = run;
        for (int w = 0; w < RS_WAVES; w++) run += cnt[w][d0 + j];
      }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < RS_ITEMS; r++) {
    if (!valid[r]) continue;
    int at = lstart[digit[r]] + rank[r];
    for (int w = 0; w < wave; w++) at += cnt[w][digit[r]];
    skey[at] = key[r];
    sval[at] = val[r];
  }
  __syncthreads();
  const int64_t tile_n = min((int64_t)RS_TILE, n - (int64_t)blockIdx.x * RS_TILE);
#pragma unroll
  for (int r = 0; r < RS_ITEMS; r++) {
    const int pos = r * RS_THREADS + threadIdx.x;
    if (pos >= tile_n) continue;
    const u64 k = skey[pos];
    const unsigned d = (unsigned)(k >> shift) & mask;
    const int at = base[d] + (pos - lstart[d]);
    kout[at] = k;
    vout[at] = sval[pos];
  }
}

// Up to RS1_MAX pairs: one workgroup takes them through every digit without leaving LDS
// (sort_block.h), one launch instead of three per digit.
constexpr int RS1_ITEMS = 4, RS1_MAX = RS1_THREADS * RS1_ITEMS;
__global__ __launch_bounds__(RS1_THREADS) void k_rs_single(const u64 *__restrict__ kin, const int *__restrict__ vin,
                                                           u64 *__restrict__ kout, int *__restrict__ vout, int n,
                                                           int end_bit, int width, const int *__restrict__ n_dev) {
  constexpr int ITEMS = RS1_ITEMS;
  if (n_dev) n = *n_dev;
  __shared__ BlockSort<ITEMS> sh;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int q0 = wave * (ITEMS * 64);
  u64 key[ITEMS];
  int val[ITEMS];
  bool valid[ITEMS];
#pragma unroll
  for (int r = 0; r < ITEMS; r++) {
    const int i = q0 + r * 64 + lane;
    valid[r] = i < n;
    key[r] = valid[r] ? kin[i] : 0ull;
    val[r] = valid[r] ? vin[i] : 0;
  }
  block_sort<ITEMS>(sh, key, val, valid, end_bit, width);
  for (int i = threadIdx.x; i < n; i += RS1_THREADS) {
    kout[i] = sh.skey[i];
    vout[i] = sh.sval[i];
  }
}

// n_dev (optional): the number of pairs, on the device; n is then an upper bound that sizes the
// launches, and tiles past the real end find nothing to do.
void radix_sort_pairs(Metadata &m, const u64 *kin, u64 *kout, const int *vin, int *vout, int64_t n, int end_bit,
                      hipStream_t s, const int *n_dev) {
  if (n <= 0) return;
  end_bit = std::max(1, std::min(64, end_bit));
  if (n >= ((int64_t)1 << 31)) throw Error("sort: too many pairs");
  // as few digits as RS_MAX_BITS bits each allow, of equal width
  const int passes = (end_bit + RS_MAX_BITS - 1) / RS_MAX_BITS;
  const int width = (end_bit + passes - 1) / passes;
  if (n <= RS1_MAX) {
    const int p1 = (end_bit + RS1_BITS - 1) / RS1_BITS;
    k_rs_single<<<dim3(1), RS1_THREADS, 0, s>>>(kin, vin, kout, vout, (int)n, end_bit, (end_bit + p1 - 1) / p1, n_dev);
    LAUNCH_CHECK();
    return;
  }
  // Large inputs take tiles of 4096 pairs (longer runs per digit value in the scatter's stores: a
  // million pairs of 35 bits 145 -> 122 us, eight million 800 -> 490 us); below half a million pairs
  // there are too few of those to fill the chip and smaller tiles are faster, down to 512 pairs
  // (30 bits: 88 000 pairs 64 -> 55 us, 15 000 pairs 60 -> 44 us, 150 000 pairs 72 -> 61 us with 1024).
  const int items = n >= 500000 ? 16 : n >= 300000 ? 8 : n >= 120000 ? 4 : 2;
  const int tile = RS_THREADS * items;
  const int tiles = (int)ceil_div(n, tile);
  // scratch: a second pair of arrays (when there is more than one pass), the tile counts, the totals
  const size_t kbytes = round_up((size_t)n * sizeof(u64), 256), vbytes = round_up((size_t)n * sizeof(int), 256);
  const size_t hbytes = round_up(((size_t)1 << width) * tiles * sizeof(int), 256);
  m.tmp.reserve((passes > 1 ? kbytes + vbytes : 0) + hbytes + ((size_t)1 << width) * sizeof(int));
  unsigned char *p = m.tmp.p;
  u64 *ktmp = nullptr;
  int *vtmp = nullptr;
  if (passes > 1) {
    ktmp = reinterpret_cast<u64 *>(p);
    vtmp = reinterpret_cast<int *>(p + kbytes);
    p += kbytes + vbytes;
  }
  int *hist = reinterpret_cast<int *>(p), *tot = reinterpret_cast<int *>(p + hbytes);
  const u64 *ksrc = kin;
  const int *vsrc = vin;
  for (int pass = 0; pass < passes; pass++) {
    // the last pass writes the output arrays; the ones before alternate so that it can
    const bool to_out = (passes - 1 - pass) % 2 == 0;
    u64 *kdst = to_out ? kout : ktmp;
    int *vdst = to_out ? vout : vtmp;
    const int shift = width * pass, bits = std::min(width, end_bit - shift);
    switch (items) {
#define RS_PASS(I)                                                                                                  \
  case I:                                                                                                           \
    k_rs_hist<I><<<dim3(tiles), RS_THREADS *(I >= 4 ? 4 : I), 0, s>>>(ksrc, n, shift, bits, tiles, hist, n_dev);    \
    LAUNCH_CHECK();                                                                                                 \
    k_rs_colscan<<<dim3(1 << bits), 64, 0, s>>>(hist, tiles, tot);                                                  \
    LAUNCH_CHECK();                                                                                                 \
    k_rs_scatter<I><<<dim3(tiles), RS_THREADS, 0, s>>>(ksrc, vsrc, kdst, vdst, n, shift, bits, tiles, hist, tot, n_dev); \
    LAUNCH_CHECK();                                                                                                 \
    break;
      RS_PASS(16)
      RS_PASS(8)
      RS_PASS(4)
      RS_PASS(2)
#undef RS_PASS
    default:
      throw Error("sort: internal tile size");
    }
    ksrc = kdst;
    vsrc = vdst;
  }
}

}  // namespace scn
