// Levels, input-layer rules and rulebook construction on the GPU.
//
// The reference builds all of this on the host, one hash map per sample, one thread per
// sample (Metadata/IOLayersRules.h:18-121, Metadata/SubmanifoldConvolutionRules.h:26-87,
// Metadata/ConvolutionRules.h:11-105).  Here every step is data-parallel over sites:
//   * sites are packed into 64-bit keys (common.h) and radix-sorted; equal keys become
//     adjacent, which yields duplicate groups (input layer), the distinct output sites of
//     a strided convolution, and a spatially coherent row schedule, all without atomics;
//   * neighbours are found through a block-occupancy grid: one table entry per block of 64
//     consecutive key values (occupancy mask + rank of its first site), so the taps of a
//     filter box mostly re-use the entry of the previous tap;
//   * rules are stored output-stationary as a table nbr[tap][position] instead of
//     per-tap pair lists; pair lists are produced on demand by ballot/prefix compaction.
#include <cstring>

#include <rocprim/rocprim.hpp>
#include "sort_block.h"

#include <algorithm>

#include "metadata.h"

namespace scn {

static const int TB = 256;
static inline dim3 grid_for(int64_t n, int tb = TB) { return dim3((unsigned)std::max<int64_t>(1, ceil_div(n, tb))); }

SizeKey mk(int dim, const int64_t *a, const int64_t *b, const int64_t *c) {
  SizeKey k(a, a + dim);
  if (b) k.insert(k.end(), b, b + dim);
  if (c) k.insert(k.end(), c, c + dim);
  return k;
}

Geom make_geom(int dim, const int64_t *spatial) {
  Geom g{};
  g.dim = dim;
  g.vol = 1;
  int bits = 1;
  for (int d = 0; d < dim; d++) {
    if (spatial[d] < 1 || spatial[d] > (int64_t)1 << 30) throw Error("spatial size out of range");
    g.size[d] = spatial[d];
    while (((int64_t)1 << bits) < spatial[d]) bits++;
    if (dim >= 4) {
      if (g.vol > ((int64_t)1 << 62) / spatial[d]) throw Error("spatial volume does not fit a 64-bit site key");
      g.vol *= spatial[d];
    }
  }
  g.bits = bits;
  if (dim <= 3) {
    if ((dim == 3 && bits > 21) || (dim == 2 && bits > 31) || dim * bits > 62)
      throw Error("spatial size too large for the site key");
    int free_bits = 63 - dim * bits;
    g.max_batch = free_bits >= 31 ? ((int64_t)1 << 31) - 1 : (int64_t)1 << free_bits;
  } else {
    g.max_batch = std::min<int64_t>(((int64_t)1 << 31) - 1, ((int64_t)1 << 62) / g.vol);
  }
  return g;
}

// Number of low key bits that can be non-zero for sample indices below `batch`.
static int key_bits(const Geom &g, int64_t batch) {
  auto bitlen = [](uint64_t v) {
    int b = 0;
    while (v) {
      b++;
      v >>= 1;
    }
    return b;
  };
  batch = std::max<int64_t>(batch, 1);
  if (g.dim <= 3) return g.dim * g.bits + bitlen((uint64_t)batch - 1);
  return bitlen((uint64_t)batch * (uint64_t)g.vol - 1);
}

// ---- small utilities -------------------------------------------------------------------

void wait_for_consumers(Metadata &m, hipStream_t s) {
  if (!m.consumer_known || m.consumer == s) return;
  hipEvent_t ev;
  HIP_CHECK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
  HIP_CHECK(hipEventRecord(ev, m.consumer));
  HIP_CHECK(hipStreamWaitEvent(s, ev, 0));
  HIP_CHECK(hipEventDestroy(ev));  // released once it has completed
}

static void settle_lookups(Metadata &m, const SizeKey &size, hipStream_t s);
static const int COUNT_SLOTS = 32;  // copies of a rulebook's per-tap counters (a power of two)

__global__ void k_fill32(uint32_t *p, uint32_t v, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}
// 16 bytes per store: p is 16-byte aligned, n4 counts groups of four words
__global__ void k_fill128(uint4 *p, uint32_t v, int64_t n4) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const uint4 vv = make_uint4(v, v, v, v);
  for (; i < n4; i += stride) p[i] = vv;
}
void fill32(void *p, uint32_t v, int64_t n, hipStream_t s) {
  if (n <= 0) return;
  if (n >= 4096 && (uintptr_t)p % 16 == 0) {  // large fills: wide stores, the tail word by word
    const int64_t n4 = n / 4;
    k_fill128<<<dim3((unsigned)std::min<int64_t>(ceil_div(n4, TB), 256 * 32)), TB, 0, s>>>((uint4 *)p, v, n4);
    LAUNCH_CHECK();
    p = (uint32_t *)p + n4 * 4;
    n -= n4 * 4;
    if (n == 0) return;
  }
  int64_t blocks = std::min<int64_t>(ceil_div(n, TB), 256 * 32);
  k_fill32<<<dim3((unsigned)blocks), TB, 0, s>>>((uint32_t *)p, v, n);
  LAUNCH_CHECK();
}

// Three fills in one launch (a strided rulebook starts from two empty tables and zeroed
// counts; at the deep levels of a network every launch saved is time saved).  blockIdx.y
// picks the buffer; sizes in words, all multiples of four on 16-byte aligned buffers, else
// three separate fills.
struct Fill3 {
  uint4 *p[3];
  uint32_t v[3];
  int64_t n4[3];
};
__global__ void k_fill3(Fill3 f) {
  const int b = blockIdx.y;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const uint4 vv = make_uint4(f.v[b], f.v[b], f.v[b], f.v[b]);
  for (; i < f.n4[b]; i += stride) f.p[b][i] = vv;
}
static void fill3(void *p0, uint32_t v0, int64_t n0, void *p1, uint32_t v1, int64_t n1, void *p2, uint32_t v2,
                  int64_t n2, hipStream_t s) {
  void *p[3] = {p0, p1, p2};
  const uint32_t v[3] = {v0, v1, v2};
  const int64_t n[3] = {n0, n1, n2};
  bool wide = true;
  for (int b = 0; b < 3; b++) wide = wide && n[b] > 0 && n[b] % 4 == 0 && (uintptr_t)p[b] % 16 == 0;
  if (!wide) {
    for (int b = 0; b < 3; b++) fill32(p[b], v[b], n[b], s);
    return;
  }
  Fill3 f;
  int64_t most = 0;
  for (int b = 0; b < 3; b++) {
    f.p[b] = (uint4 *)p[b];
    f.v[b] = v[b];
    f.n4[b] = n[b] / 4;
    most = std::max(most, f.n4[b]);
  }
  k_fill3<<<dim3((unsigned)std::min<int64_t>(ceil_div(most, TB), 256 * 32), 3), TB, 0, s>>>(f);
  LAUNCH_CHECK();
}

// Stable sort of (key, value) pairs by the low end_bit bits of the key.  From 32 k to 1.5 million pairs
// this repository's own sort (sort.hip: three short launches per digit, measured 95-145 us for a
// million pairs of 35 bits against the library's 175 us, 50-80 us against 100-150 us at 15 k to
// 250 k pairs); above, the library's radix sort, whose tiles stage their pairs through LDS and
// write long runs (measured faster from about two million pairs on).
using RadixAlways = rocprim::radix_sort_config<rocprim::default_config, rocprim::default_config,
                                               rocprim::default_config, 4096>;
static void sort_pairs(Metadata &m, const unsigned long long *kin, unsigned long long *kout,
                       const int *vin, int *vout, int64_t n, hipStream_t s, int end_bit = 64) {
  if ((n > 32768 && n <= 1500000) || n <= 4096) {  // up to 4096 pairs: one launch, one workgroup
    radix_sort_pairs(m, kin, kout, vin, vout, n, end_bit, s);
    return;
  }
  size_t bytes = 0;
  if (n <= 32768) {  // rocPRIM's own choice at this size (a merge sort of a few passes) is the fastest measured
    HIP_CHECK(rocprim::radix_sort_pairs(nullptr, bytes, kin, kout, vin, vout, (size_t)n, 0u, (unsigned)end_bit, s));
    m.tmp.reserve(bytes + 16);
    HIP_CHECK(rocprim::radix_sort_pairs(m.tmp.p, bytes, kin, kout, vin, vout, (size_t)n, 0u, (unsigned)end_bit, s));
    return;
  }
  HIP_CHECK(rocprim::radix_sort_pairs<RadixAlways>(nullptr, bytes, kin, kout, vin, vout, (size_t)n, 0u,
                                                   (unsigned)end_bit, s));
  m.tmp.reserve(bytes + 16);
  HIP_CHECK(rocprim::radix_sort_pairs<RadixAlways>(m.tmp.p, bytes, kin, kout, vin, vout, (size_t)n, 0u,
                                                   (unsigned)end_bit, s));
}
// Exclusive prefix sums of one or two int arrays in two launches that wait for nothing (no
// look-back between workgroups): k_scan_tiles sums every tile of SCAN_TILE elements, k_scan_write
// adds up the tile sums in front of its tile (a few hundred at most per million elements) and scans
// the tile's own elements inside the workgroup.  gridDim.y picks the array.
constexpr int SCAN_THREADS = 1024, SCAN_TILE = 4 * SCAN_THREADS;
struct ScanJobs {
  const int *in[2];
  int *out[2];
  int64_t n[2];
  int *tile_sums[2];
};
__device__ inline void scan_load(const int *in, int64_t n, int64_t i0, int (&v)[4]) {
  if (i0 + 4 <= n) {
    const int4 q = *reinterpret_cast<const int4 *>(in + i0);
    v[0] = q.x, v[1] = q.y, v[2] = q.z, v[3] = q.w;
  } else {
    for (int i = 0; i < 4; i++) v[i] = i0 + i < n ? in[i0 + i] : 0;
  }
}
__global__ __launch_bounds__(SCAN_THREADS) void k_scan_tiles(ScanJobs j) {
  const int a = blockIdx.y;
  const int64_t n = j.n[a], i0 = (int64_t)blockIdx.x * SCAN_TILE + 4 * threadIdx.x;
  if ((int64_t)blockIdx.x * SCAN_TILE >= n) return;
  __shared__ int total;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  int v[4];
  scan_load(j.in[a], n, i0, v);
  int sum = v[0] + v[1] + v[2] + v[3];
#pragma unroll
  for (int o = 32; o; o >>= 1) sum += __shfl_xor(sum, o, 64);
  if ((threadIdx.x & 63) == 0 && sum) atomicAdd(&total, sum);
  __syncthreads();
  if (threadIdx.x == 0) j.tile_sums[a][blockIdx.x] = total;
}
__global__ __launch_bounds__(SCAN_THREADS) void k_scan_write(ScanJobs j) {
  const int a = blockIdx.y;
  const int64_t n = j.n[a], i0 = (int64_t)blockIdx.x * SCAN_TILE + 4 * threadIdx.x;
  if ((int64_t)blockIdx.x * SCAN_TILE >= n) return;
  __shared__ int part[SCAN_THREADS / 64], wave_sum[SCAN_THREADS / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int before = 0;
  for (int i = threadIdx.x; i < (int)blockIdx.x; i += SCAN_THREADS) before += j.tile_sums[a][i];
#pragma unroll
  for (int o = 32; o; o >>= 1) before += __shfl_xor(before, o, 64);
  int v[4];
  scan_load(j.in[a], n, i0, v);
  const int mine = v[0] + v[1] + v[2] + v[3];
  int incl = mine;  // inclusive prefix over the wavefront's lanes
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  if (lane == 63) wave_sum[wave] = incl;
  if (lane == 0) part[wave] = before;
  __syncthreads();
  int run = incl - mine;
  for (int w = 0; w < SCAN_THREADS / 64; w++) run += part[w] + (w < wave ? wave_sum[w] : 0);
  int *out = j.out[a];
  if (i0 + 4 <= n) {
    int4 q;
    q.x = run, q.y = run + v[0], q.z = run + v[0] + v[1], q.w = run + v[0] + v[1] + v[2];
    *reinterpret_cast<int4 *>(out + i0) = q;
  } else {
    for (int i = 0; i < 4 && i0 + i < n; i++) {
      out[i0 + i] = run;
      run += v[i];
    }
  }
}
// in_b == nullptr: one array.  The arrays start at 16-byte boundaries (whole buffers of the pool).
static void exclusive_scan(Metadata &m, const int *in_a, int *out_a, int64_t n_a, hipStream_t s, const int *in_b = nullptr,
                           int *out_b = nullptr, int64_t n_b = 0) {
  const int64_t most = std::max(n_a, n_b);
  if (most <= 0) return;
  const int tiles = (int)ceil_div(most, SCAN_TILE);
  m.scan_tiles.reserve(2 * (size_t)tiles);
  ScanJobs j;
  j.in[0] = in_a, j.out[0] = out_a, j.n[0] = n_a, j.tile_sums[0] = m.scan_tiles.p;
  j.in[1] = in_b, j.out[1] = out_b, j.n[1] = in_b ? n_b : 0, j.tile_sums[1] = m.scan_tiles.p + tiles;
  const dim3 grid((unsigned)tiles, in_b ? 2 : 1);
  k_scan_tiles<<<grid, SCAN_THREADS, 0, s>>>(j);
  LAUNCH_CHECK();
  k_scan_write<<<grid, SCAN_THREADS, 0, s>>>(j);
  LAUNCH_CHECK();
}
// Copies `words` ints from the device into the handle's pinned words and waits for them: the
// one host round trip of a construction step.
static const int *fetch_words(Metadata &m, const int *dev, int words, hipStream_t s) {
  if (words > Metadata::PINNED_WORDS) throw Error("internal: read-back larger than the pinned words");
  if (!m.pinned) m.pinned = static_cast<int *>(pinned_acquire(Metadata::PINNED_WORDS * sizeof(int)));
  HIP_CHECK(hipMemcpyAsync(m.pinned, dev, words * sizeof(int), hipMemcpyDeviceToHost, s));
  HIP_CHECK(hipStreamSynchronize(s));
  return m.pinned;
}
template <class T> static T read_back(const T *dev, hipStream_t s) {
  T h;
  HIP_CHECK(hipMemcpyAsync(&h, dev, sizeof(T), hipMemcpyDeviceToHost, s));
  HIP_CHECK(hipStreamSynchronize(s));
  return h;
}

static void alloc_level(Level &l, const Geom &g, int64_t n, int batch) {
  l.g = g;
  l.n = n;
  l.npad = round_up(std::max<int64_t>(n, 1), 64);
  l.batch = batch;
  l.coords.reserve((size_t)(g.dim + 1) * l.npad);
  l.keys.reserve((size_t)l.npad);
  l.grid_built = false;
}

// ---- input layer -----------------------------------------------------------------------

// A maximum over the whole grid without hammering one address: wavefront shuffle, one LDS
// atomic per wavefront, then one global atomic per workgroup into one of 64 slots (a cache line
// apart), and only when it can raise the slot (the plain read may be stale, which costs an
// atomic that changes nothing).  20 000 same-address atomics cost ~130 us on a 1.3 M-point
// input, this costs ~10.  Every thread of the workgroup must call it; values <= floor are
// not reported.  The host takes the maximum over the slots.
static const int MAX_SLOTS = 64, MAX_SLOT_STRIDE = 16;
__device__ inline void grid_max(int v, int floor, int *slots) {
  __shared__ int block_max;
  if (threadIdx.x == 0) block_max = floor;
  __syncthreads();
  for (int off = 32; off; off >>= 1) v = max(v, __shfl_xor(v, off));
  if ((threadIdx.x & 63) == 0 && v > floor) atomicMax(&block_max, v);
  __syncthreads();
  int *slot = slots + MAX_SLOT_STRIDE * (blockIdx.x & (MAX_SLOTS - 1));
  if (threadIdx.x == 0 && block_max > floor && block_max > __builtin_nontemporal_load(slot)) atomicMax(slot, block_max);
}

// Adds up a count over a whole grid of workgroups with no launch in front to clear a counter and
// none behind to add up: every workgroup adds (1 << 32 | its count) to *ticket, so the value a
// workgroup gets back tells it how many came before and what they counted; the last one writes
// the sum to ticket[1] and puts the ticket back to zero for the next launch.  Every thread of
// every workgroup must call it, once.  Launches that share a ticket must not overlap (one stream).
// Same-address atomics take about 12 ns each: grids of a few hundred workgroups (COUNT_GRID) that
// stride over their input, not one workgroup per 256 elements.
static const int COUNT_GRID = 256;
__device__ inline void grid_count(int mine, unsigned long long *ticket) {
  __shared__ int block_total;
  if (threadIdx.x == 0) block_total = 0;
  __syncthreads();
#pragma unroll
  for (int o = 32; o; o >>= 1) mine += __shfl_xor(mine, o, 64);
  if ((threadIdx.x & 63) == 0 && mine) atomicAdd(&block_total, mine);
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned long long old = atomicAdd(ticket, (1ull << 32) | (unsigned long long)(unsigned)block_total);
    if ((old >> 32) == gridDim.x - 1) {
      ticket[1] = (old & 0xFFFFFFFFull) + (unsigned)block_total;
      atomicExch(ticket, 0ull);
    }
  }
}
static dim3 count_grid(int64_t n) { return dim3((unsigned)std::max<int64_t>(1, std::min<int64_t>(ceil_div(n, TB), COUNT_GRID))); }
static unsigned long long *count_ticket(Metadata &m, hipStream_t s) {
  if (!m.ticket.p) {
    m.ticket.reserve(2);
    fill32(m.ticket.p, 0, 4, s);
  }
  return m.ticket.p;
}

// flags[0] |= 1: coordinate outside the grid; |= 2: sample index out of range.
// bl_len > 0: the sample of point i is i / bl_len and a negative first coordinate marks an
// empty position (Metadata/IOLayersRules.h:183,204,234): key EMPTY, counted in flags[4].
__global__ void k_input_keys(Geom g, CoordSrc coords, int64_t n, int ncols, int64_t bl_len,
                             unsigned long long *keys, int *idx, int *flags) {
  // flags[0]: error bits, flags[4]: empty positions, flags[8...]: slots of the largest sample index
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int bmax = 0;
  bool empty = false;
  if (i < n) {
    const int64_t c0 = i * ncols;
    int cc[SCN_MAXD];
    bool ok = true;
    empty = bl_len > 0 && coord_at(coords, c0) < 0;
    for (int d = 0; d < g.dim; d++) {
      int64_t v = coord_at(coords, c0 + d);
      if (v < 0 || v >= g.size[d]) ok = false;
      cc[d] = (int)v;
    }
    int64_t b = bl_len > 0 ? i / bl_len : (ncols > g.dim ? coord_at(coords, c0 + g.dim) : 0);
    if (b < 0 || b >= g.max_batch) {
      atomicOr(&flags[0], 2);
      ok = false;
      b = 0;
    }
    if (empty) {
      keys[i] = SCN_EMPTY_KEY;
    } else if (!ok) {
      atomicOr(&flags[0], 1);
      keys[i] = SCN_EMPTY_KEY;
    } else {
      keys[i] = site_key(g, cc, (int)b);
    }
    idx[i] = (int)i;
    bmax = (int)b;
  }
  grid_max(bmax, 0, flags + 8);
  const unsigned long long em = __ballot(empty);
  if ((threadIdx.x & 63) == 0 && em) atomicAdd(&flags[4], __popcll(em));
}

// mode 0: row = input index.
__global__ void k_input_rows_identity(Geom g, CoordSrc coords, int64_t n, int ncols, int64_t bl_len,
                                      int64_t npad, int *soa) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t c0 = i * ncols;
  for (int d = 0; d < g.dim; d++) soa[d * npad + i] = (int)coord_at(coords, c0 + d);
  soa[g.dim * npad + i] = bl_len > 0 ? (int)(i / bl_len) : (ncols > g.dim ? (int)coord_at(coords, c0 + g.dim) : 0);
}

// After the stable sort: head[p] marks the first point of each group of equal keys;
// is_first[i] marks input points that are the first occurrence of their site.  Positions from
// n_valid on hold the empty points of a batch-by-length input: no group, never first.
__global__ void k_group_heads(const unsigned long long *skeys, const int *sidx, int64_t n, int64_t n_valid,
                              int *head, int *is_first) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p == n) head[p] = 0;  // one element past the end, so that a scan of n + 1 ends with the total
  if (p >= n) return;
  int h = (p < n_valid && (p == 0 || skeys[p] != skeys[p - 1])) ? 1 : 0;
  head[p] = h;
  is_first[sidx[p]] = h;
}

// Row = rank of the first occurrence in input order (Metadata/IOLayersRules.h:84-87).
// Two passes so that every array is written in ascending order (stream compaction) instead of
// being scattered: one over the sorted points for what is indexed by group (key order) ...
__global__ void k_assign_groups(const int *sidx, const int *head, const int *head_scan, const int *first_scan,
                                const unsigned long long *sorted_keys, int64_t n, int *sched, int *row_of_group,
                                int *head_pos, unsigned long long *pos_keys) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n || !head[p]) return;
  const int row = first_scan[sidx[p]];
  const int u = head_scan[p];
  sched[u] = row;
  pos_keys[u] = sorted_keys[p];  // the level's keys by schedule position (Level::skeys)
  row_of_group[u] = row;
  head_pos[u] = (int)p;
}
// ... and one over the points in input order for what is indexed by row: coordinates and key
// of every first occurrence.
__global__ void k_assign_coords(Geom g, CoordSrc coords, int ncols, int64_t bl_len, const int *is_first,
                                const int *first_scan, int64_t n, int64_t npad, int *soa,
                                unsigned long long *level_keys) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n || !is_first[i]) return;
  const int row = first_scan[i];
  const int64_t c0 = i * ncols;
  int cc[SCN_MAXD];
  for (int d = 0; d < g.dim; d++) {
    cc[d] = (int)coord_at(coords, c0 + d);
    soa[d * npad + row] = cc[d];
  }
  const int b = bl_len > 0 ? (int)(i / bl_len) : (ncols > g.dim ? (int)coord_at(coords, c0 + g.dim) : 0);
  soa[g.dim * npad + row] = b;
  level_keys[row] = site_key(g, cc, b);
}

__global__ void k_finish_groups(const int *sidx, const int *head, const int *head_scan,
                                const int *row_of_group, const int *head_pos, int64_t n,
                                int n_groups, int *row_of_input, int *run_start, int *run_len,
                                int *max_active) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int len = 0;
  if (p < n) {
    int u = head_scan[p] + head[p] - 1;
    int row = row_of_group[u];
    row_of_input[sidx[p]] = row;
    if (head[p]) {
      int next = (u + 1 < n_groups) ? head_pos[u + 1] : (int)n;
      len = next - (int)p;
      run_start[row] = (int)p;
      run_len[row] = len;
    }
  }
  grid_max(len, 1, max_active);  // longest run; runs of one are the floor
}

void build_input_layer(Metadata &m, const int64_t *spatial, CoordSrc coords, int64_t n,
                       int ncols, int min_batch, int mode, hipStream_t s, int64_t bl_length,
                       const unsigned char *overwrite) {
  const bool bl = bl_length > 0;
  if (bl ? ncols != m.dim : (ncols != m.dim && ncols != m.dim + 1))
    throw Error(bl ? "coords must be [batch, length, dim]" : "coords must have dim or dim+1 columns");
  if (mode < 0 || mode > 5 || (mode == 5 && bl)) throw Error("input layer mode must be 0..4");
  if (mode == 5 && !overwrite) mode = 1;  // nothing overwrites: every site keeps its first point
  if (n >= ((int64_t)1 << 31) - 64) throw Error("too many input points for int32 rule indices");
  Geom g = make_geom(m.dim, spatial);
  SizeKey key = mk(m.dim, spatial);
  m.input_size = key;
  if (m.levels.count(key)) settle_lookups(m, key, s);
  Level &L = m.levels[key];
  InputRules &R = m.input;
  // Metadata/IOLayersRules.h:96-107 against :180-205: the plain layer lists the first point of
  // a site in mode 1 and the last in mode 2, the batch-by-length layer the other way round.
  R.user_mode = mode;
  R.mode = (bl && (mode == 1 || mode == 2)) ? 3 - mode : mode;
  R.n_in = n;
  R.max_active = 1;
  R.bl_length = bl_length;
  R.bl_batch = bl ? n / bl_length : 0;
  int batch_floor = bl ? (int)R.bl_batch : (ncols == m.dim ? 1 : std::max(min_batch, 0));
  m.builds++;
  if (n == 0) {
    alloc_level(L, g, 0, batch_floor);
    L.identity_sched = true;
    R.n_out = 0;
    return;
  }
  m.k0.reserve(n);
  m.k1.reserve(n);
  m.v0.reserve(n);
  m.v1.reserve(n);
  const int n_flags = 8 + MAX_SLOTS * MAX_SLOT_STRIDE;
  m.dflags.reserve(n_flags);
  fill32(m.dflags.p, 0, n_flags, s);
  k_input_keys<<<grid_for(n), TB, 0, s>>>(g, coords, n, ncols, bl_length, m.k0.p, m.v0.p, m.dflags.p);
  LAUNCH_CHECK();
  const int *fetched = fetch_words(m, m.dflags.p, n_flags, s);
  release_staging(m);  // coordinates from the host: their copies are behind us now
  const std::vector<int> hflags(fetched, fetched + n_flags);
  if (hflags[0] & 2) throw Error("input layer: sample index negative or too large for the site key");
  if (hflags[0] & 1) throw Error("input layer: coordinate outside [0, spatial_size)");
  int top_batch = 0;
  for (int i = 0; i < MAX_SLOTS; i++) top_batch = std::max(top_batch, hflags[8 + i * MAX_SLOT_STRIDE]);
  const int64_t n_empty = hflags[4], nv = n - n_empty;
  if (n_empty && mode == 0) throw Error("batch-by-length input layer: mode 0 needs every position filled");
  // only the key bits that samples 0..top_batch can set take part in the sort; one bit more
  // keeps the EMPTY keys (all ones) of empty positions behind every real key
  const int bits = key_bits(g, (int64_t)top_batch + 1) + (n_empty ? 1 : 0);
  if (bits > 64) throw Error("batch-by-length input layer: grid too large for a layer with empty positions");
  // Metadata/IOLayersRules.h:25,46-47,76-77: the batch is at least min_batch and grows to
  // the largest sample index + 1; without a sample column there is exactly one sample.
  // :140 batch-by-length: one grid per sample of the input, filled or not.
  int batch = bl ? batch_floor : (ncols == m.dim ? 1 : std::max(batch_floor, top_batch + 1));

  if (mode == 0) {
    alloc_level(L, g, n, batch);
    L.sched.reserve(n);
    L.skeys.reserve(n + 1);
    L.identity_sched = false;
    L.dups = true;  // mode 0 does not merge repeated points
    // the sorted pairs are the level's schedule and its positions' keys
    sort_pairs(m, m.k0.p, L.skeys.p, m.v0.p, L.sched.p, n, s, bits);
    L.skeys_ready = true;
    k_input_rows_identity<<<grid_for(n), TB, 0, s>>>(g, coords, n, ncols, bl_length, L.npad, L.coords.p);
    LAUNCH_CHECK();
    HIP_CHECK(hipMemcpyAsync(L.keys.p, m.k0.p, n * sizeof(unsigned long long), hipMemcpyDeviceToDevice, s));
    R.n_out = n;
    return;
  }
  sort_pairs(m, m.k0.p, m.k1.p, m.v0.p, m.v1.p, n, s, bits);

  m.f0.reserve(n + 1);  // head
  m.f1.reserve(n);  // is_first
  m.s0.reserve(n + 1);  // head_scan
  m.s1.reserve(n + 1);  // first_scan
  k_group_heads<<<grid_for(n + 1), TB, 0, s>>>(m.k1.p, m.v1.p, n, nv, m.f0.p, m.f1.p);
  LAUNCH_CHECK();
  // head[n] = 0: the last element of its scan is the number of groups; both scans in one pair of launches
  exclusive_scan(m, m.f0.p, m.s0.p, n + 1, s, m.f1.p, m.s1.p, n);
  const int64_t N = fetch_words(m, m.s0.p + n, 1, s)[0];
  alloc_level(L, g, N, batch);
  L.sched.reserve(N);
  L.identity_sched = false;
  R.n_out = N;
  R.row_of_input.reserve(n);
  R.sorted_idx.reserve(n);
  R.run_start.reserve(std::max<int64_t>(N, 1));
  R.run_len.reserve(std::max<int64_t>(N, 1));
  if (n_empty) fill32(R.row_of_input.p, 0xFFFFFFFFu, n, s);  // empty positions belong to no row
  HIP_CHECK(hipMemcpyAsync(R.sorted_idx.p, m.v1.p, n * sizeof(int), hipMemcpyDeviceToDevice, s));
  if (mode == 5) {  // the caller's flags are read again by every forward pass: keep a copy
    R.overwrite.reserve(n);
    HIP_CHECK(hipMemcpyAsync(R.overwrite.p, overwrite, n, hipMemcpyDeviceToDevice, s));
  }
  if (N == 0) return;
  m.v0.reserve(std::max<int64_t>(n, 2 * N + 2));  // reused: row_of_group | head_pos
  int *row_of_group = m.v0.p, *head_pos = m.v0.p + N;
  R.max_slots.reserve(MAX_SLOTS * MAX_SLOT_STRIDE);
  fill32(R.max_slots.p, 0, MAX_SLOTS * MAX_SLOT_STRIDE, s);
  L.skeys.reserve(N + 1);
  k_assign_groups<<<grid_for(nv), TB, 0, s>>>(m.v1.p, m.f0.p, m.s0.p, m.s1.p, m.k1.p, nv, L.sched.p, row_of_group, head_pos,
                                              L.skeys.p);
  L.skeys_ready = true;
  LAUNCH_CHECK();
  k_assign_coords<<<grid_for(n), TB, 0, s>>>(g, coords, ncols, bl_length, m.f1.p, m.s1.p, n, L.npad, L.coords.p,
                                             L.keys.p);
  LAUNCH_CHECK();
  // the groups end where the empty positions begin
  k_finish_groups<<<grid_for(nv), TB, 0, s>>>(m.v1.p, m.f0.p, m.s0.p, row_of_group, head_pos, nv, (int)N,
                                              R.row_of_input.p, R.run_start.p, R.run_len.p,
                                              R.max_slots.p);
  LAUNCH_CHECK();
  // Metadata/IOLayersRules.h:92,111: maxActive is 1 for modes 1 and 2, the longest run for the
  // summing modes (runs of one never touch the slots).  Only the rule export asks for it, so
  // it stays on the device until then (input_max_active): one host round trip less per scene.
  R.max_active = 1;
  R.max_known = !(mode == 3 || mode == 4);
}
int input_max_active(Metadata &m) {
  InputRules &R = m.input;
  if (!R.max_known) {
    // a rare call (rule export): wait for the whole device rather than keep the construction's stream alive
    std::vector<int> h((size_t)MAX_SLOTS * MAX_SLOT_STRIDE);
    HIP_CHECK(hipDeviceSynchronize());
    HIP_CHECK(hipMemcpy(h.data(), R.max_slots.p, h.size() * sizeof(int), hipMemcpyDeviceToHost));
    for (int i = 0; i < MAX_SLOTS; i++) R.max_active = std::max(R.max_active, h[i * MAX_SLOT_STRIDE]);
    R.max_known = true;
  }
  return R.max_active;
}

// Reference layout of the rule rows (Metadata/IOLayersRules.h:96-119).
__global__ void k_export_input_rules(const int *sorted_idx, const int *run_start, const int *run_len,
                                     const unsigned char *overwrite, int64_t n_out, int mode, int max_active,
                                     int *rows) {
  int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= n_out) return;
  int *o = rows + r * (1 + max_active);
  int st = run_start[r], len = run_len[r];
  if (mode == 1 || mode == 2 || mode == 5) {
    o[0] = 1;
    o[1] = listed_point(sorted_idx, st, len, mode, overwrite);
  } else {
    o[0] = len;
    for (int q = 0; q < max_active; q++) o[1 + q] = q < len ? sorted_idx[st + q] : 0;
  }
}
void export_input_rules(Metadata &m, int *rows, hipStream_t s) {
  InputRules &R = m.input;
  if (R.mode <= 0 || R.n_out == 0) return;
  k_export_input_rules<<<grid_for(R.n_out), TB, 0, s>>>(R.sorted_idx.p, R.run_start.p, R.run_len.p,
                                                        R.overwrite.p, R.n_out, R.mode, input_max_active(m), rows);
  LAUNCH_CHECK();
}

__global__ void k_locations(const int *soa, int64_t n, int64_t npad, int dim, int64_t *out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * (dim + 1)) return;
  int64_t r = i / (dim + 1);
  int d = (int)(i - r * (dim + 1));
  out[i] = soa[d * npad + r];
}
void spatial_locations(Metadata &m, const int64_t *spatial, int64_t *out, hipStream_t s) {
  auto it = m.levels.find(mk(m.dim, spatial));
  if (it == m.levels.end() || it->second.n == 0) return;
  Level &L = it->second;
  k_locations<<<grid_for(L.n * (m.dim + 1)), TB, 0, s>>>(L.coords.p, L.n, L.npad, m.dim, out);
  LAUNCH_CHECK();
}

// ---- site lookup of a level -------------------------------------------------------------

// skey[t] = key of the row at schedule position t (ascending).
__global__ void k_sorted_keys(const unsigned long long *keys, const int *sched, int64_t n,
                              unsigned long long *skey) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) skey[t] = keys[sched ? sched[t] : t];
}
// Levels whose keys may repeat (an input layer that does not merge points): the distinct sites are
// the runs of equal keys in schedule order; ukey[u], urow[u] for the u-th of them, where the last
// row of its run wins (Metadata/IOLayersRules.h:41,54: repeated `mp[p] = i`), and head[u] = 1 where a
// block of 64 keys starts.  Two launches, with no scan between them: a workgroup
// takes SITE_TILE consecutive positions (four per thread), k_site_tails counts the distinct
// sites of every tile, k_site_compact adds up the tiles in front of its own, numbers its sites
// with a prefix inside the workgroup, writes ukey / urow / head and counts the blocks
// (grid_count); *last_site = the index of the last distinct site.
constexpr int SITE_THREADS = 1024, SITE_TILE = 4 * SITE_THREADS;
__global__ __launch_bounds__(SITE_THREADS) void k_site_tails(const unsigned long long *skey, int64_t n, int *tile_sites) {
  __shared__ int total;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  const int64_t t0 = (int64_t)blockIdx.x * SITE_TILE + 4 * threadIdx.x;
  int mine = 0;
  for (int i = 0; i < 4; i++) {
    const int64_t t = t0 + i;
    mine += (t < n && (t == n - 1 || skey[t + 1] != skey[t])) ? 1 : 0;
  }
#pragma unroll
  for (int o = 32; o; o >>= 1) mine += __shfl_xor(mine, o, 64);
  if ((threadIdx.x & 63) == 0 && mine) atomicAdd(&total, mine);
  __syncthreads();
  if (threadIdx.x == 0) tile_sites[blockIdx.x] = total;
}
__global__ __launch_bounds__(SITE_THREADS) void k_site_compact(const unsigned long long *skey, const int *sched, int64_t n,
                                                               const int *tile_sites, unsigned long long *ukey,
                                                               int *urow, int *head, unsigned long long *ticket,
                                                               int *last_site) {
  __shared__ int part[SITE_THREADS / 64], wave_sites[SITE_THREADS / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int before = 0;
  for (int i = threadIdx.x; i < (int)blockIdx.x; i += SITE_THREADS) before += tile_sites[i];
#pragma unroll
  for (int o = 32; o; o >>= 1) before += __shfl_xor(before, o, 64);
  const int64_t t0 = (int64_t)blockIdx.x * SITE_TILE + 4 * threadIdx.x;
  bool tail[4];
  int mine = 0;
  for (int i = 0; i < 4; i++) {
    const int64_t t = t0 + i;
    tail[i] = t < n && (t == n - 1 || skey[t + 1] != skey[t]);
    mine += tail[i] ? 1 : 0;
  }
  int incl = mine;  // inclusive prefix over the wavefront's lanes
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  if (lane == 63) wave_sites[wave] = incl;
  if (lane == 0) part[wave] = before;
  __syncthreads();
  int u = incl - mine;
  for (int w = 0; w < SITE_THREADS / 64; w++) u += part[w] + (w < wave ? wave_sites[w] : 0);
  int heads = 0;
  for (int i = 0; i < 4; i++) {
    if (!tail[i]) continue;
    const int64_t t = t0 + i;
    const unsigned long long k = skey[t];
    int64_t j = t;  // first position of the site's run: the key in front of it is the previous site's
    while (j > 0 && skey[j - 1] == k) j--;
    const int h = (j == 0 || (skey[j - 1] >> 6) != (k >> 6)) ? 1 : 0;
    ukey[u] = k;
    urow[u] = sched ? sched[t] : (int)t;
    head[u] = h;
    heads += h;
    u++;
  }
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == SITE_THREADS - 1) *last_site = u - 1;
  grid_count(heads, ticket);
}
// The size of a level's block table is decided on the device (no host round trip): from the
// number of blocks, capacity = the power of two >= 4 * blocks (at least 64), within what is
// allocated (room for twice as many blocks as there are sites).  A wavefront of a rule kernel waits
// for the longest of its lanes' probe sequences: a table a quarter to an eighth full keeps those short.
__device__ inline unsigned long long grid_capacity(long long nblocks, long long cap_alloc) {
  unsigned long long cap = 64;
  while (cap < (unsigned long long)nblocks * 4ull && cap < (unsigned long long)cap_alloc) cap <<= 1;
  return cap;
}
// skey[t] = key of the row at schedule position t; head[t] = 1 where a block of 64 keys starts;
// ticket[1] = the number of blocks (grid_count).
__global__ void k_grid_heads(const unsigned long long *keys, const int *sched, int64_t n,
                             unsigned long long *skey, int *head, unsigned long long *ticket) {
  int heads = 0;
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (int64_t)gridDim.x * blockDim.x) {
    const unsigned long long k = keys[sched ? sched[t] : t];
    skey[t] = k;
    const int h = (t == 0 || (k >> 6) != (keys[sched ? sched[t - 1] : t - 1] >> 6)) ? 1 : 0;
    head[t] = h;
    heads += h;
  }
  grid_count(heads, ticket);
}
// n_sites_dev: the index of the last distinct site when their number is only known on the device
// (levels with repeated keys; positions behind it hold stale keys), else null.
__global__ void k_block_heads(const unsigned long long *ukey, int64_t n, const int *n_sites_dev, int *head,
                              unsigned long long *ticket) {
  const int64_t U = n_sites_dev ? (int64_t)*n_sites_dev + 1 : n;
  int heads = 0;
  for (int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; u < U; u += (int64_t)gridDim.x * blockDim.x) {
    const int h = (u == 0 || (ukey[u] >> 6) != (ukey[u - 1] >> 6)) ? 1 : 0;
    head[u] = h;
    heads += h;
  }
  grid_count(heads, ticket);
}
// Empties the part of the table that will be used and records its mask (capacity - 1) for the
// kernels that follow.  ticket[1]: the number of blocks, as the head kernel in front left it.
// zero (optional): words the caller wants cleared in the same launch (a rulebook's counters).
__global__ void k_block_clear(BlockEntry *table, int64_t cap_alloc, const unsigned long long *ticket,
                              unsigned long long *mask_out, uint32_t *zero, int zero_words) {
  int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t i = b; i < zero_words; i += (int64_t)gridDim.x * blockDim.x) zero[i] = 0u;
  const unsigned long long cap = grid_capacity((long long)ticket[1], cap_alloc);
  if (b == 0) *mask_out = cap - 1;
  if (b < cap_alloc && (unsigned long long)b < cap) {
    table[b].key = SCN_EMPTY_KEY;
    table[b].mask = 0ull;
    table[b].base = 0;
  }
}
// One lane per distinct site (ascending keys).  The sites of a block are neighbours in that order,
// so a wavefront ORs the occupancy bits of each run of equal block keys it holds with six
// shuffle steps; the first lane of a run claims the block's slot (or finds it, when the run began
// in the wavefront before and that one was faster) and ORs the run's bits in; the lane that
// starts the block (head) also stores its rank.  k_block_clear has zeroed the bits.
__global__ void k_block_insert(const unsigned long long *ukey, const int *head, int64_t n_sites,
                               const int *n_sites_dev, BlockEntry *table, const unsigned long long *mask_p) {
  const int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t U = n_sites_dev ? (int64_t)*n_sites_dev + 1 : n_sites;
  const int lane = threadIdx.x & 63;
  const bool live = u < U;
  const unsigned long long k = live ? ukey[u] : 0ull;
  // dead lanes (behind the last site) get a block key no live lane has
  const unsigned long long bkey = live ? k >> 6 : SCN_EMPTY_KEY;
  unsigned long long bits = live ? 1ull << (k & 63) : 0ull;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const unsigned long long other_bits = __shfl_down(bits, o, 64);
    const unsigned long long other_key = __shfl_down(bkey, o, 64);
    if (lane + o < 64 && other_key == bkey) bits |= other_bits;
  }
  const unsigned long long before = __shfl_up(bkey, 1, 64);
  if (!live || (lane > 0 && before == bkey)) return;  // not the first lane of its run
  const unsigned long long mask = *mask_p;
  unsigned long long b = hash64(bkey) & mask;
  for (unsigned long long i = 0; i <= mask; i++) {
    const unsigned long long old = atomicCAS(&table[b].key, SCN_EMPTY_KEY, bkey);
    if (old == SCN_EMPTY_KEY || old == bkey) {
      atomicOr(&table[b].mask, bits);
      if (head[u]) table[b].base = (int)u;
      return;
    }
    b = (b + 1) & mask;
  }
}

// skeys[t] = key of the site at schedule position t (ascending), computed once per level.
static const unsigned long long *position_keys(Level &L, hipStream_t s) {
  if (!L.skeys_ready && L.n) {
    L.skeys.reserve(L.n + 1);
    k_sorted_keys<<<grid_for(L.n), TB, 0, s>>>(L.keys.p, L.sched_ptr(), L.n, L.skeys.p);
    LAUNCH_CHECK();
    L.skeys_ready = true;
  }
  return L.skeys.p;
}

// zero / zero_words: see k_block_clear; false when the table was there already and nothing was cleared.
static bool ensure_grid(Metadata &m, Level &L, hipStream_t s, void *zero = nullptr, int zero_words = 0) {
  if (L.grid_built) return false;
  const int64_t n = L.n;
  L.skeys.reserve(n + 1);
  m.k1.reserve(n + 1);
  m.f0.reserve(n + 1);
  m.s0.reserve(n + 1);
  L.gridp.reserve(2);
  // every site could be a block of its own: room for that, of which only the part the
  // device-side capacity covers is ever touched
  uint64_t cap_alloc = 64;
  while (cap_alloc < (uint64_t)n * 2) cap_alloc <<= 1;
  L.table.reserve(cap_alloc);
  const unsigned long long *ukey = L.skeys.p;
  const int *n_sites_dev = nullptr;
  unsigned long long *ticket = count_ticket(m, s);
  if (n) {
    if (L.dups) {
      // distinct sites first: ukey / urow by compaction; their number stays on the device
      position_keys(L, s);
      const int tiles = (int)ceil_div(n, SITE_TILE);
      m.f1.reserve(tiles);
      m.s1.reserve(1);
      L.urow.reserve(n);
      k_site_tails<<<dim3(tiles), SITE_THREADS, 0, s>>>(L.skeys.p, n, m.f1.p);
      LAUNCH_CHECK();
      k_site_compact<<<dim3(tiles), SITE_THREADS, 0, s>>>(L.skeys.p, L.sched_ptr(), n, m.f1.p, m.k1.p, L.urow.p, m.f0.p,
                                                         ticket, m.s1.p);
      LAUNCH_CHECK();
      n_sites_dev = m.s1.p;  // index of the last distinct site
      ukey = m.k1.p;
    } else if (L.skeys_ready) {  // the input layer left the positions' keys
      k_block_heads<<<count_grid(n), TB, 0, s>>>(L.skeys.p, n, nullptr, m.f0.p, ticket);
      LAUNCH_CHECK();
    } else {
      k_grid_heads<<<count_grid(n), TB, 0, s>>>(L.keys.p, L.sched_ptr(), n, L.skeys.p, m.f0.p, ticket);
      LAUNCH_CHECK();
    }
  } else {
    fill32(ticket + 1, 0, 2, s);  // no sites: no blocks
  }
  k_block_clear<<<grid_for((int64_t)cap_alloc), TB, 0, s>>>(L.table.p, (int64_t)cap_alloc, ticket, L.gridp.p,
                                                            static_cast<uint32_t *>(zero), zero_words);
  LAUNCH_CHECK();
  if (n) {
    k_block_insert<<<grid_for(n), TB, 0, s>>>(ukey, m.f0.p, n, n_sites_dev, L.table.p, L.gridp.p);
    LAUNCH_CHECK();
  }
  L.grid_built = true;
  L.skeys_ready = n > 0;
  return true;
}

// ---- submanifold rules -----------------------------------------------------------------

struct Filt {
  int dim, K, M;
  int size[SCN_MAXD], stride[SCN_MAXD], out_size[SCN_MAXD], m[SCN_MAXD];
  // tap k of the site c of a position reads c * stride + k - off: off = size / 2 for a submanifold
  // filter (stride 1, centred), 0 for a strided one read from its coarse side
  int off[SCN_MAXD];
};

// One thread per schedule position t: probe the filter box around the row's site
// (Metadata/SubmanifoldConvolutionRules.h:11-45; taps enumerate the box row-major with the
// last dimension fastest, Metadata/RectangularRegions.h:56-71).
// The positions may also be those of the coarse level of a strided filter (soa, sched, n, npad
// describe them) and g, table, urow the fine level its taps are looked up in
// (Metadata/ConvolutionRules.h:19-31 read from the output side): f.stride and f.off say which.
// dup_keys (levels whose keys may repeat, else null): the positions' keys, ascending; of a run of
// equal keys only the last position is a site (`mp[p] = i`, Metadata/IOLayersRules.h:41,54), the
// others are rows no rule touches.
__global__ void k_subm_rules(Geom g, Filt f, const int *soa, const int *sched, int64_t n,
                             int64_t npad, const BlockEntry *table, const unsigned long long *mask_p,
                             const int *urow, int *nbr, unsigned long long *counts, int parts,
                             const unsigned long long *dup_keys) {
  const unsigned long long mask = *mask_p;
  // blockDim = 64 * parts: wavefront p of the block handles taps [p*K/parts, (p+1)*K/parts)
  // (one slice of the first filter dimension) of the block's 64 positions.
  extern __shared__ int lcount[];
  for (int k = threadIdx.x; k < f.K; k += blockDim.x) lcount[k] = 0;
  __syncthreads();
  const int part = threadIdx.x >> 6;
  int64_t t = (int64_t)blockIdx.x * 64 + (threadIdx.x & 63);
  const bool live = t < n;
  if (!live) t = n - 1;  // idle lanes shadow the last position so that ballots see whole wavefronts
  {
    int row = sched ? sched[t] : (int)t;
    int c[SCN_MAXD], tap[SCN_MAXD], q[SCN_MAXD];
    const int per = f.K / parts;
    const int k0 = part * per;
    {
      int r = k0;
      for (int d = g.dim - 1; d >= 0; d--) {
        tap[d] = r % f.size[d];
        r /= f.size[d];
      }
    }
    for (int d = 0; d < g.dim; d++) c[d] = soa[d * npad + row];
    int b = soa[g.dim * npad + row];
    unsigned long long last_bkey = SCN_EMPTY_KEY, last_mask = 0;  // block of the previous tap
    int last_base = 0;
    const bool shadowed = dup_keys && t + 1 < n && dup_keys[t + 1] == dup_keys[t];
    for (int k = k0; k < k0 + per; k++) {
      bool inside = !shadowed;
      for (int d = 0; d < g.dim; d++) {
        q[d] = c[d] * f.stride[d] + tap[d] - f.off[d];
        if (q[d] < 0 || q[d] >= g.size[d]) inside = false;
      }
      int j = -1;
      if (inside) {
        const unsigned long long key = site_key(g, q, b);
        const unsigned long long bkey = key >> 6;
        if (bkey != last_bkey) {
          last_bkey = bkey;
          const int64_t slot = block_find(table, mask, bkey);
          last_mask = slot >= 0 ? table[slot].mask : 0ull;
          last_base = slot >= 0 ? table[slot].base : 0;
        }
        const unsigned long long bit = 1ull << (key & 63);
        if (last_mask & bit) {
          const int r = last_base + __popcll(last_mask & (bit - 1));
          j = urow ? urow[r] : r;
        }
      }
      if (live) nbr[(int64_t)k * npad + t] = j;
      const unsigned long long hits = __ballot(live && j >= 0);
      if ((threadIdx.x & 63) == 0 && hits) atomicAdd(&lcount[k], __popcll(hits));
      for (int d = g.dim - 1; d >= 0; d--) {  // next tap, last dimension fastest
        if (++tap[d] < f.size[d]) break;
        tap[d] = 0;
      }
    }
  }
  __syncthreads();
  unsigned long long *slot = counts + (size_t)(blockIdx.x & (COUNT_SLOTS - 1)) * f.K;
  for (int k = threadIdx.x; k < f.K; k += blockDim.x)
    if (lcount[k]) atomicAdd(&slot[k], (unsigned long long)lcount[k]);
}

// ---- pattern-sorted positions ----------------------------------------------------------

// Positions are re-sorted by neighbour pattern inside PATTERN_WINDOWS equal ranges of the
// space-filling-curve order.  A convolution workgroup takes consecutive positions, so after
// the sort its rows share one or two patterns: it walks only the taps those patterns have and
// every 16-row granule is busy on each of them.  One range per XCD (workgroups are dealt to
// XCDs in contiguous ranges) keeps an XCD's gathers inside one compact region of space;
// measured on room scenes of 60k..4M sites, 8 or 16 ranges beat both 256-position blocks
// (by 20-30% for 64..256 channels) and one global sort (which loses the locality).
static const int PATTERN_WINDOWS = 8;
// Below this many positions the sort runs over the whole table (Table::spread).  A level of
// 250 k sites or fewer is a few waves of workgroups: what decides a kernel's duration there is how
// evenly the expensive tiles (those with the most taps) are spread over the CUs and how early they
// start, not L2 locality.  One window puts them first, kernels then deal tiles to workgroups in
// turn; it also wastes fewer MFMAs on 16-row granules of mixed patterns (13 % -> 5 % at 60 k sites,
// 37 % -> 17 % at 14 k).  Measured on the room scene: convolutions 9 % faster at 247 k sites, 19 %
// at 61 k, 9 % at 14 k; at a million sites one window is slower.
static const int64_t PATTERN_WHOLE_BELOW = 300000;

// Sort key of a position: window, then the number of absent taps (shifted right by pc_shift
// when the key bits are short), then the tap mask, or, when the mask has more than code_bits
// bits, a hash of it (positions with the same taps still end up next to each other, but
// patterns that share a hash value interleave and similar patterns are no longer neighbours:
// measured 2 % slower convolutions on a 27-tap table, so only filters of more than 27 taps get
// one).  Inside a window the positions with the most taps come first and the cheapest last,
// which shortens the tail of kernels that hand positions out in order.
// masks[t] (K <= 32): the tap mask itself, for the granule masks.
// Tables of up to 32 taps: the code is the mask's rank in the order (most taps first, then by
// value), which sorts exactly like count-then-mask does in K bits instead of K + log2(K): three
// passes instead of four for 27 taps, one instead of two for 8 or 9.
struct PatternKey {  // how finalize_table's sort key is put together
  int64_t window;
  int pc_bits, pc_shift, code_bits, K, ranked;
};
struct Binomials {
  unsigned v[33][33];      // v[i][j] = C(i, j)
  unsigned above[33][33];  // above[K][c] = number of K-bit masks with more than c set bits
  constexpr Binomials() : v{}, above{} {
    for (int i = 0; i < 33; i++) {
      v[i][0] = 1;
      for (int j = 1; j <= i; j++) v[i][j] = v[i - 1][j - 1] + (j < i ? v[i - 1][j] : 0u);
    }
    for (int k = 0; k < 33; k++)
      for (int c = k - 1; c >= 0; c--) above[k][c] = above[k][c + 1] + v[k][c + 1];
  }
};
__constant__ const Binomials c_binom = Binomials();
// Rank of a K-bit mask (K <= 32) among all K-bit masks ordered by falling number of set bits, then
// rising value: the masks with more bits come first, and among those with c bits the rank is the
// combinatorial number, the sum over the set bits of C(position, number of set bits up to and
// including it) (one independent table read per bit).
__device__ inline unsigned mask_rank(unsigned mask, int K) {
  unsigned r = c_binom.above[K][__popc(mask)];
  for (int i = 0; i < K; i++)
    if (mask >> i & 1u) r += c_binom.v[i][__popc(mask & ((2u << i) - 1u))];
  return r;
}
// The same with the number of taps known to the compiler: every table read is issued before the
// first is waited for (the loop above waits for one after the other, which a kernel with few
// wavefronts to switch to pays in full).
template <int K> __device__ inline unsigned mask_rank_fixed(unsigned mask) {
  unsigned r = c_binom.above[K][__popc(mask)];
#pragma unroll
  for (int i = 0; i < K; i++) {
    const unsigned term = c_binom.v[i][__popc(mask & ((2u << i) - 1u))];  // read whether the bit is set or not
    r += (mask >> i & 1u) ? term : 0u;
  }
  return r;
}
// window_of: t / window without the 64-bit division (there are at most PATTERN_WINDOWS windows).
__device__ inline unsigned window_of(int64_t t, int64_t window) {
  unsigned w = 0;
#pragma unroll
  for (int i = 1; i < PATTERN_WINDOWS; i++) w += t >= i * window ? 1u : 0u;
  return w;
}
template <int KC = 0>
__device__ inline unsigned long long pattern_key(const PatternKey &p, int64_t t, unsigned long long mask) {
  unsigned long long hi = window_of(t, p.window);
  if (p.ranked) return (hi << p.code_bits) | (KC > 0 ? mask_rank_fixed<(KC > 0 ? KC : 1)>((unsigned)mask) : mask_rank((unsigned)mask, p.K));
  if (p.pc_bits) hi = (hi << p.pc_bits) | (unsigned long long)((p.K - __popcll(mask)) >> p.pc_shift);
  const unsigned long long code = p.code_bits < p.K ? (mask * 0x9E3779B97F4A7C15ull) >> (64 - p.code_bits) : mask;
  return (hi << p.code_bits) | code;
}
__global__ void k_table_masks(PatternKey pk, const int *nbr, int K, int64_t n, int64_t npad, unsigned long long *keys,
                              int *idx, unsigned *masks) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  unsigned long long mask = 0;
  for (int k = 0; k < K; k++)
    if (nbr[(int64_t)k * npad + t] >= 0) mask |= 1ull << k;
  keys[t] = pattern_key(pk, t, mask);
  idx[t] = (int)t;
  if (masks) masks[t] = (unsigned)mask;
}
__global__ void k_table_permute(const int *nbr, int K, int64_t n, int64_t npad, const int *perm,
                                const int *base, int *nbr2, int *rowmap) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * K) return;
  int k = (int)(i / n);
  int64_t t = i - (int64_t)k * n;
  int src = perm[t];
  nbr2[(int64_t)k * npad + t] = nbr[(int64_t)k * npad + src];
  if (k == 0) rowmap[t] = base ? base[src] : src;
}
// Few taps (K <= 16): one thread moves a position's K entries and the granule masks come out of
// the same launch (an OR over the 16 lanes of a granule).
__global__ void k_table_permute_few(const int *nbr, int K, int64_t n, int64_t npad, const int *perm, const int *base,
                                    int *nbr2, int *rowmap, unsigned *gmask) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  unsigned mk = 0;
  if (t < n) {
    const int src = perm[t];
    for (int k = 0; k < K; k++) {
      const int v = nbr[(int64_t)k * npad + src];
      nbr2[(int64_t)k * npad + t] = v;
      mk |= v >= 0 ? 1u << k : 0u;
    }
    rowmap[t] = base ? base[src] : src;
  }
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) mk |= __shfl_xor(mk, o, 64);
  if ((threadIdx.x & 15) == 0 && t < n) gmask[t >> 4] = mk;
}
// The same from a site-major table rows[src][ROWW]: a workgroup moves 64 positions, reading
// each one's row in 16-byte pieces and writing 256 contiguous bytes per tap.
template <int ROWW>
__global__ __launch_bounds__(256) void k_table_rows_permute(const int *__restrict__ rows, int K, int64_t n, int64_t npad,
                                                            const int *__restrict__ perm, const int *__restrict__ base,
                                                            int *__restrict__ nbr2, int *__restrict__ rowmap,
                                                            unsigned *__restrict__ gmask) {
  __shared__ int tile[64][ROWW + 1];
  const int64_t t0 = (int64_t)blockIdx.x * 64;
  for (int e = threadIdx.x; e < 64 * (ROWW / 4); e += 256) {
    const int r = e / (ROWW / 4), c = 4 * (e % (ROWW / 4));
    if (t0 + r >= n) break;
    const int4 v = *reinterpret_cast<const int4 *>(rows + (int64_t)perm[t0 + r] * ROWW + c);
    tile[r][c + 0] = v.x;
    tile[r][c + 1] = v.y;
    tile[r][c + 2] = v.z;
    tile[r][c + 3] = v.w;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < K * 64; e += 256) {
    const int k = e >> 6, r = e & 63;
    if (t0 + r < n) nbr2[(int64_t)k * npad + t0 + r] = tile[r][k];
  }
  if (threadIdx.x < 64) {  // the first wavefront
    const bool live = t0 + threadIdx.x < n;
    if (live) {
      const int src = perm[t0 + threadIdx.x];
      rowmap[t0 + threadIdx.x] = base ? base[src] : src;
    }
    // gmask of the workgroup's four granules: OR of the tap masks of 16 positions each
    unsigned mk = 0;
    if (live)
      for (int k = 0; k < K; k++) mk |= tile[threadIdx.x][k] >= 0 ? 1u << k : 0u;
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) mk |= __shfl_xor(mk, o, 64);
    if ((threadIdx.x & 15) == 0 && t0 + threadIdx.x < n) gmask[(t0 + threadIdx.x) >> 4] = mk;
  }
}
// gmask[i] = OR of the tap masks of granule i's 16 positions; perm[t] = the position's place before the sort
__global__ void k_granule_masks(const unsigned *masks, const int *perm, int64_t n, int64_t n_granules, unsigned *gmask) {
  int64_t gi = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gi >= n_granules) return;
  unsigned m = 0;
  for (int r = 0; r < 16; r++) {
    const int64_t t = gi * 16 + r;
    if (t < n) m |= masks[perm[t]];
  }
  gmask[gi] = m;
}
__global__ void k_copy_rowmap(const int *base, int64_t n, int *rowmap) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) rowmap[t] = base ? base[t] : (int)t;
}

// t.nbr is indexed by the level's schedule (base[t] = row, or t itself when base is null).
// Re-sort positions by neighbour pattern inside windows and record the position -> row map.
// The sort key's layout for a table of n positions and K taps (K <= 62).
static PatternKey pattern_plan(int64_t n, int K, int &key_bits) {
  PatternKey p;
  p.K = K;
  p.window = std::max<int64_t>(256, round_up(ceil_div(n, n < PATTERN_WHOLE_BELOW ? 1 : PATTERN_WINDOWS), 256));
  int block_bits = 0;
  while (((int64_t)1 << block_bits) < ceil_div(n, p.window)) block_bits++;
  p.ranked = K <= 32;
  if (p.ranked) {
    p.pc_bits = p.pc_shift = 0;
    p.code_bits = K;
    key_bits = K + block_bits;
    return p;
  }
  // Wider filters (33 .. 62 taps): count of absent taps, then the mask.  Up to 40 key bits (four
  // sort passes): beyond that the count gives way first, then the mask (hashed).  Measured on
  // 27-tap tables of a million rows before those were ranked: no count at all costs 2.5-4 % in
  // every convolution (the heaviest positions no longer come first), a 14-bit hash of the mask 4-7 %.
  int pc_bits = 1;
  while ((1 << pc_bits) <= K) pc_bits++;
  const int budget = 40;
  p.pc_shift = std::max(0, std::min(pc_bits, block_bits + pc_bits + K - budget));
  p.pc_bits = pc_bits - p.pc_shift;
  p.code_bits = std::min(K, budget - block_bits - p.pc_bits);
  key_bits = p.code_bits + p.pc_bits + block_bits;
  return p;
}
// Buffers the keyed form of finalize_table expects to be filled: m.k0 keys, m.v0 positions, m.f1 masks.
static void reserve_pattern_buffers(Metadata &m, const Table &t) {
  m.k0.reserve(t.n);
  m.k1.reserve(t.n);
  m.v0.reserve(t.n);
  m.v1.reserve(t.n);
  if (t.K <= 32) m.f1.reserve(t.n);
}
// keyed: the kernel that wrote the table has written the sort keys, positions and masks as well.
// rows (with keyed): that kernel wrote the table site-major, roww ints per site, into `rows`
// and t.nbr is still empty.
static void finalize_table(Metadata &m, Table &t, const int *base, hipStream_t s, bool keyed = false,
                           const int *rows = nullptr, int roww = 0) {
  if (t.n == 0) {
    t.identity_rows = true;
    return;
  }
  t.rowmap.reserve(t.npad);
  if (t.K > 62) {  // the pattern does not fit a machine word: keep schedule order
    t.identity_rows = base == nullptr;
    if (base) {
      k_copy_rowmap<<<grid_for(t.n), TB, 0, s>>>(base, t.n, t.rowmap.p);
      LAUNCH_CHECK();
    }
    return;
  }
  int key_bits = 0;
  const PatternKey pk = pattern_plan(t.n, t.K, key_bits);
  t.spread = pk.window >= t.n;
  reserve_pattern_buffers(m, t);
  unsigned *masks = t.K <= 32 ? reinterpret_cast<unsigned *>(m.f1.p) : nullptr;
  if (!keyed) {
    k_table_masks<<<grid_for(t.n), TB, 0, s>>>(pk, t.nbr.p, t.K, t.n, t.npad, m.k0.p, m.v0.p, masks);
    LAUNCH_CHECK();
  }
  sort_pairs(m, m.k0.p, m.k1.p, m.v0.p, m.v1.p, t.n, s, key_bits);
  DevBuf<int> nbr2;
  nbr2.reserve((size_t)t.K * t.npad);
  const bool few = !rows && t.K <= 16;
  const bool from_rows = (rows && (roww == 32 || roww == 12)) || few;  // these also write the granule masks (K <= 32)
  if (from_rows) t.gmask.reserve(ceil_div(t.n, 16));
  if (rows && roww == 32)
    k_table_rows_permute<32><<<grid_for(t.n, 64), 256, 0, s>>>(rows, t.K, t.n, t.npad, m.v1.p, base, nbr2.p, t.rowmap.p,
                                                               t.gmask.p);
  else if (rows && roww == 12)
    k_table_rows_permute<12><<<grid_for(t.n, 64), 256, 0, s>>>(rows, t.K, t.n, t.npad, m.v1.p, base, nbr2.p, t.rowmap.p,
                                                               t.gmask.p);
  else if (few)
    k_table_permute_few<<<grid_for(t.n), TB, 0, s>>>(t.nbr.p, t.K, t.n, t.npad, m.v1.p, base, nbr2.p, t.rowmap.p,
                                                     t.gmask.p);
  else
    k_table_permute<<<grid_for(t.n * t.K), TB, 0, s>>>(t.nbr.p, t.K, t.n, t.npad, m.v1.p, base, nbr2.p,
                                                       t.rowmap.p);
  LAUNCH_CHECK();
  t.nbr = std::move(nbr2);
  t.identity_rows = false;
  if (t.K <= 32 && !from_rows) {
    const int64_t n_granules = ceil_div(t.n, 16);
    t.gmask.reserve(n_granules);
    k_granule_masks<<<grid_for(n_granules), TB, 0, s>>>(masks, m.v1.p, t.n, n_granules, t.gmask.p);
    LAUNCH_CHECK();
  }
}

// Filter 3 in every dimension, dim 2 or 3 (the common case): the Morton key of a neighbour
// is the OR of per-coordinate spread values, so each coordinate is spread three times per
// site (for c-1, c, c+1) instead of once per tap, and the tap loop is fully unrolled.
// One wavefront per slice of the first filter dimension, as in k_subm_rules.
// HALF: the same filter at stride 2, looked up from the coarse side (Metadata/ConvolutionRules.h:19-31
// read backwards): the positions are the sites of the coarse level (keys of pos_bits bits per
// coordinate), the site c of one has the taps 2c, 2c+1, 2c+2 per dimension in level g, whose
// table this is.
#define S3_ROW_INTS(dim) ((dim) == 3 ? 32 : 12)  // ints per site of the site-major table: 27 or 9 taps, padded to 16 bytes
template <int DIM, bool HALF>
__global__ void k_subm_rules_s3(Geom g, int pos_bits, const unsigned long long *skeys, int64_t n, int64_t npad,
                                const BlockEntry *table, const unsigned long long *mask_p, const int *urow,
                                int *rows, unsigned long long *counts, PatternKey pk, unsigned long long *pkeys,
                                int *pidx, unsigned *pmasks, bool dups) {
  const unsigned long long mask = *mask_p;
  constexpr int K = DIM == 3 ? 27 : 9;
  constexpr int PER = K / 3;
  constexpr int ROWW = S3_ROW_INTS(DIM);
  // The table leaves this kernel site-major, rows[t][ROWW] (taps K .. ROWW-1 = -1): the
  // pattern sort moves whole sites, and k_table_rows_permute then reads one contiguous row per
  // site where a tap-major table would be read four bytes per sector.
  __shared__ int tile[64][ROWW + 1];
  __shared__ int lcount[K];
  __shared__ unsigned lmask[64];  // tap mask of each of the block's positions, collected from the three wavefronts
  if (threadIdx.x < K) lcount[threadIdx.x] = 0;
  if (threadIdx.x < 64) lmask[threadIdx.x] = 0;
  __syncthreads();
  const int part = threadIdx.x >> 6;  // offset -1, 0, +1 along the first dimension
  // Workgroups are dealt to the eight XCDs in turn; XCD x takes the x-th eighth of the positions
  // (a compact piece of the curve), so that the block entries it looks up, an eighth of the
  // table, stay in its own L2.
  const int per_xcd = gridDim.x / 8;  // the grid is a multiple of eight workgroups
  const int wg = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if ((int64_t)wg * 64 >= n) return;  // the whole workgroup: padding of the grid
  int64_t t = (int64_t)wg * 64 + (threadIdx.x & 63);
  const bool live = t < n;
  if (!live) t = n - 1;
  // The site of position t from its key (the positions' keys are one coalesced read; the
  // coordinates by row would be four gathers through the schedule, per wavefront).
  const unsigned long long skey = skeys[t];
  // keys may repeat (dups): only the last position of a run of equal keys is a site, see k_subm_rules
  const bool shadowed = dups && t + 1 < n && skeys[t + 1] == skey;
  unsigned long long sp[DIM][3];
  bool okc[DIM][3];
  int cd[DIM];
#pragma unroll
  for (int d = 0; d < DIM; d++) {
    const int c = DIM == 3 ? (int)compact3(skey >> (DIM - 1 - d)) & ((1 << pos_bits) - 1)
                           : (int)compact2(skey >> (DIM - 1 - d)) & ((1 << pos_bits) - 1);
    cd[d] = HALF ? 2 * c + 1 : c;  // the middle tap's coordinate in level g
#pragma unroll
    for (int o = 0; o < 3; o++) {
      const int v = cd[d] + o - 1;
      okc[d][o] = v >= 0 && v < g.size[d];
    }
    // The three coordinates' bits in place in a key of level g, without spreading them: the middle
    // one's are the position's own (moved up one bit per coordinate and with the low bit set for the
    // coarse side of a stride-2 filter: 2c + 1), and one more or less is an add or a subtract that
    // carries across the other coordinates' bit positions (filled with ones for the add; the
    // subtract borrows through their zeros).  A coordinate that leaves [0, 2^bits) gives a wrong
    // pattern, and is out of range: okc is false for it.
    constexpr unsigned long long EVERY = DIM == 3 ? 0x1249249249249249ull : 0x5555555555555555ull;
    const int sh = DIM - 1 - d;
    const unsigned long long md = (EVERY & ((1ull << (DIM * g.bits)) - 1ull)) << sh, one = 1ull << sh;
    unsigned long long mid;
    if (HALF)
      mid = ((skey & ((EVERY & ((1ull << (DIM * pos_bits)) - 1ull)) << sh)) << DIM) | one;
    else
      mid = skey & md;
    sp[d][1] = mid;
    sp[d][0] = HALF ? mid & ~one : (mid - one) & md;
    sp[d][2] = ((mid | ~md) + one) & md;
  }
  const unsigned long long bpart = (skey >> (DIM * pos_bits)) << (DIM * g.bits);  // the sample index, in its place in level g's keys
  // The lane's taps (first-dimension offset fixed by its wavefront) lie in at most two blocks
  // along each remaining dimension: the blocks of the lowest and of the highest in-range
  // coordinate.  All of them (two, or two by two) are looked up at once, whole 32-byte entries,
  // so that a lane waits for memory once instead of once per block it meets on its way through
  // the taps; entry e = 2 * (high block along dimension 1) + (high block along the last).
  constexpr int NE = DIM == 3 ? 4 : 2;
  constexpr int SH = DIM == 3 ? 2 : 3;  // a block is 4 x 4 x 4 sites, or 8 x 8
  bool hi_of[DIM][3];  // [d][o]: tap offset o along d lies in the high block (always false when there is only one)
  unsigned long long lo_sp[DIM], hi_sp[DIM];
  bool split[DIM];
#pragma unroll
  for (int d = 1; d < DIM; d++) {
    const int lo = max(cd[d] - 1, 0), hi = min(cd[d] + 1, g.size[d] - 1);
    split[d] = (lo >> SH) != (hi >> SH);
    lo_sp[d] = okc[d][0] ? sp[d][0] : sp[d][1];
    hi_sp[d] = okc[d][2] ? sp[d][2] : sp[d][1];
#pragma unroll
    for (int o = 0; o < 3; o++) hi_of[d][o] = ((cd[d] + o - 1) >> SH) != (lo >> SH);
  }
  unsigned long long ebits[NE];
  int ebase[NE];
  {
    unsigned long long want[NE], at[NE];
    ulonglong2 km[NE];
    bool need[NE];
#pragma unroll
    for (int e = 0; e < NE; e++) {
      unsigned long long key;
      if (DIM == 3) {
        key = bpart | sp[0][part] | ((e & 2) ? hi_sp[1] : lo_sp[1]) | ((e & 1) ? hi_sp[2] : lo_sp[2]);
        need[e] = okc[0][part] && (!(e & 2) || split[1]) && (!(e & 1) || split[2]);
      } else {
        key = bpart | sp[0][part] | ((e & 1) ? hi_sp[1] : lo_sp[1]);
        need[e] = okc[0][part] && (!(e & 1) || split[1]);
      }
      want[e] = key >> 6;
      at[e] = hash64(want[e]) & mask;
    }
#pragma unroll
    for (int e = 0; e < NE; e++) {
      km[e] = make_ulonglong2(SCN_EMPTY_KEY, 0ull);
      ebase[e] = 0;
      if (need[e]) {
        km[e] = *reinterpret_cast<const ulonglong2 *>(&table[at[e]]);
        ebase[e] = table[at[e]].base;
      }
    }
#pragma unroll
    for (int e = 0; e < NE; e++) {
      ebits[e] = km[e].y;
      if (km[e].x != want[e]) {
        ebits[e] = 0ull;
        // not in its first slot: absent (empty slot), or further along the probe sequence
        if (km[e].x != SCN_EMPTY_KEY) block_lookup(table, mask, want[e], ebits[e], ebase[e]);
      }
    }
  }
  unsigned my_mask = 0;
#pragma unroll
  for (int kk = 0; kk < PER; kk++) {
    const int k = part * PER + kk;
    // taps enumerate the box with the last dimension fastest
    const int o1 = DIM == 3 ? kk / 3 : kk, o2 = kk % 3;
    bool inside;
    unsigned long long key;
    int e;
    if (DIM == 3) {
      inside = !shadowed && okc[0][part] && okc[1][o1] && okc[2][o2];
      key = bpart | sp[0][part] | sp[1][o1] | sp[2][o2];
      e = (hi_of[1][o1] ? 2 : 0) + (hi_of[2][o2] ? 1 : 0);
    } else {
      inside = !shadowed && okc[0][part] && okc[1][o1];
      key = bpart | sp[0][part] | sp[1][o1];
      e = hi_of[1][o1] ? 1 : 0;
    }
    int j = -1;
    if (inside) {
      unsigned long long bits = ebits[0];
      int base = ebase[0];
#pragma unroll
      for (int x = 1; x < NE; x++)
        if (e == x) bits = ebits[x], base = ebase[x];
      const unsigned long long bit = 1ull << (key & 63);
      if (bits & bit) {
        const int r = base + __popcll(bits & (bit - 1));
        j = urow ? urow[r] : r;
      }
    }
    tile[threadIdx.x & 63][k] = j;
    if (j >= 0) my_mask |= 1u << k;
    const unsigned long long hits = __ballot(live && j >= 0);
    if ((threadIdx.x & 63) == 0 && hits) atomicAdd(&lcount[k], __popcll(hits));
  }
  atomicOr(&lmask[threadIdx.x & 63], my_mask);
  __syncthreads();
  // the workgroup's 64 rows are one contiguous piece of the table
  for (int e = threadIdx.x; e < 64 * (ROWW / 4); e += 192) {
    const int r = e / (ROWW / 4), c = 4 * (e % (ROWW / 4));
    const int64_t tr = (int64_t)wg * 64 + r;
    if (tr >= n) break;
    int4 v;
    v.x = c + 0 < K ? tile[r][c + 0] : -1;
    v.y = c + 1 < K ? tile[r][c + 1] : -1;
    v.z = c + 2 < K ? tile[r][c + 2] : -1;
    v.w = c + 3 < K ? tile[r][c + 3] : -1;
    *reinterpret_cast<int4 *>(rows + tr * ROWW + c) = v;
  }
  unsigned long long *slot = counts + (size_t)(blockIdx.x & (COUNT_SLOTS - 1)) * K;
  if (threadIdx.x < K && lcount[threadIdx.x]) atomicAdd(&slot[threadIdx.x], (unsigned long long)lcount[threadIdx.x]);
  // what the pattern sort of finalize_table starts from (k_table_masks would re-read the table for it)
  if (threadIdx.x < 64 && live) {
    const unsigned mk = lmask[threadIdx.x];
    pkeys[t] = pattern_key<K>(pk, t, mk);
    pidx[t] = (int)t;
    pmasks[t] = mk;
  }
}

// The same rulebook for levels of up to 1024 sites (the deep levels of a network: what their
// rulebooks cost is launches, six of them on the path above), whole in one launch of one workgroup:
// the sites' keys go into a hash table in LDS (no block table is built), thread t looks the 3^d
// neighbours of position t up there, the positions are sorted by tap pattern (block_sort) and every
// thread writes its column of the finished table: taps, output row, granule masks, counts.  The
// table equals the one finalize_table makes of the same level (same keys, both sorts stable).
// COUNT (up to 256 sites, 256 threads): no sort either; the place of a position in the pattern order
// is the number of positions with a smaller key (or the same and in front of it), counted against
// all of them in LDS, which below a few hundred is faster than the passes of a radix sort.
constexpr int TINY_MAX = 1024, TINY_SLOTS = 4096, TINY_COUNT_MAX = 256;
template <int DIM, bool COUNT>
__global__ __launch_bounds__(COUNT ? TINY_COUNT_MAX : TINY_MAX) void k_subm_tiny(Geom g, const unsigned long long *skeys, const int *sched, int n,
                                                        int64_t npad, PatternKey pk, int key_bits, int width, int *nbr,
                                                        int *rowmap, unsigned *gmask, unsigned long long *counts,
                                                        int count_words) {
  constexpr int K = DIM == 3 ? 27 : 9;
  __shared__ unsigned long long hkey[TINY_SLOTS];
  __shared__ short hpos[TINY_SLOTS];
  __shared__ int lcount[K];
  __shared__ unsigned lg[TINY_MAX / 16];
  constexpr int THREADS = COUNT ? TINY_COUNT_MAX : TINY_MAX;
  const int t = threadIdx.x, lane = t & 63;
  const bool live = t < n;
  for (int i = t; i < TINY_SLOTS; i += THREADS) hkey[i] = SCN_EMPTY_KEY;
  if (t < K) lcount[t] = 0;
  if (t < TINY_MAX / 16) lg[t] = 0u;
  for (int i = t; i < count_words; i += THREADS) counts[i] = 0ull;  // every copy of the counters; copy 0 gets the counts below
  __syncthreads();
  const unsigned long long skey = live ? skeys[t] : 0ull;
  auto slot_of = [](unsigned long long key) { return (unsigned)((key * 0x9E3779B97F4A7C15ull) >> 40) & (TINY_SLOTS - 1); };
  if (live) {  // the keys of a level without repeated points are distinct
    unsigned h = slot_of(skey);
    while (atomicCAS(&hkey[h], SCN_EMPTY_KEY, skey) != SCN_EMPTY_KEY) h = (h + 1) & (TINY_SLOTS - 1);
    hpos[h] = (short)t;
  }
  __syncthreads();
  int v[K];
  unsigned mask = 0;
  {
    unsigned long long sp[DIM][3];
    bool okc[DIM][3];
#pragma unroll
    for (int d = 0; d < DIM; d++) {
      const int c = DIM == 3 ? (int)compact3(skey >> (DIM - 1 - d)) & ((1 << g.bits) - 1)
                             : (int)compact2(skey >> (DIM - 1 - d)) & ((1 << g.bits) - 1);
#pragma unroll
      for (int o = 0; o < 3; o++) {
        const int q = c + o - 1;
        okc[d][o] = q >= 0 && q < g.size[d];
        sp[d][o] = (DIM == 3 ? spread3((unsigned)q) : spread2((unsigned)q)) << (DIM - 1 - d);
      }
    }
    const unsigned long long bpart = (skey >> (DIM * g.bits)) << (DIM * g.bits);
#pragma unroll
    for (int k = 0; k < K; k++) {  // taps enumerate the box with the last dimension fastest
      const int o0 = DIM == 3 ? k / 9 : k / 3, o1 = DIM == 3 ? (k / 3) % 3 : k % 3, o2 = k % 3;
      bool inside = live && okc[0][o0] && okc[1][o1];
      unsigned long long key = bpart | sp[0][o0] | sp[1][o1];
      if (DIM == 3) {
        inside = inside && okc[DIM - 1][o2];
        key |= sp[DIM - 1][o2];
      }
      int j = -1;
      if (inside) {
        unsigned h = slot_of(key);
        for (;;) {
          const unsigned long long at = hkey[h];
          if (at == key) {
            j = hpos[h];
            break;
          }
          if (at == SCN_EMPTY_KEY) break;
          h = (h + 1) & (TINY_SLOTS - 1);
        }
      }
      v[k] = j < 0 ? -1 : (sched ? sched[j] : j);
      if (j >= 0) mask |= 1u << k;
      const unsigned long long hits = __ballot(j >= 0);
      if (lane == 0 && hits) atomicAdd(&lcount[k], __popcll(hits));
    }
  }
  unsigned long long key[1] = {live ? pattern_key<K>(pk, t, mask) : 0ull};
  int P = t;  // the position of site t in the table; threads n .. npad - 1 fill the padding
  if constexpr (COUNT) {
    __shared__ unsigned long long ckey[TINY_COUNT_MAX];
    ckey[t] = key[0];
    __syncthreads();
    int before = 0;
    for (int j = 0; j < n; j++) {
      const unsigned long long kj = ckey[j];
      before += (kj < key[0] || (kj == key[0] && j < t)) ? 1 : 0;
    }
    if (live) P = before;
  } else {
    __shared__ short pos_of[TINY_MAX];
    __shared__ BlockSort<1> sh;
    int val[1] = {t};
    const bool valid[1] = {live};
    block_sort<1>(sh, key, val, valid, key_bits, width);
    if (live) pos_of[sh.sval[t]] = (short)t;  // position t of the table holds the site sh.sval[t]
    __syncthreads();
    if (live) P = pos_of[t];
  }
  if (t < npad) {
#pragma unroll
    for (int k = 0; k < K; k++) nbr[(int64_t)k * npad + P] = live ? v[k] : -1;
  }
  if (live) {
    rowmap[P] = sched ? sched[t] : t;
    atomicOr(&lg[P >> 4], mask);
  }
  __syncthreads();
  if (t < (n + 15) / 16) gmask[t] = lg[t];
  if (t < K) counts[t] = (unsigned long long)lcount[t];
}

static Filt make_filt(int dim, const int64_t *size, const int64_t *stride, const int64_t *out_size) {
  Filt f{};
  f.dim = dim;
  int64_t K = 1, M = 1;
  for (int d = 0; d < dim; d++) {
    if (size[d] < 1 || size[d] > 64) throw Error("filter size must be in 1..64");
    f.size[d] = (int)size[d];
    f.stride[d] = stride ? (int)stride[d] : 1;
    if (f.stride[d] < 1) throw Error("filter stride must be positive");
    f.out_size[d] = out_size ? (int)out_size[d] : 0;
    f.m[d] = (f.size[d] + f.stride[d] - 1) / f.stride[d];
    f.off[d] = stride ? 0 : f.size[d] / 2;
    K *= size[d];
    M *= f.m[d];
    if (K > 4096) throw Error("filter volume above 4096 is not supported");
  }
  f.K = (int)K;
  f.M = (int)M;
  return f;
}

// Rule counts are tallied per workgroup in LDS and flushed with one atomic per tap into one of
// COUNT_SLOTS copies of the counter array (a million-site level has 15 000 workgroups; all of
// them adding to the same K addresses cost 160 us of a 700 us rulebook build).  Whoever reads
// the counts on the host sums the copies there (ensure_counts, take_macs).
static void start_counts(Table &t, hipStream_t s, bool clear = true) {
  t.cnt = std::make_shared<Counts>();
  t.cnt->K = t.K;
  t.cnt->slots = COUNT_SLOTS;
  const int64_t words = (int64_t)COUNT_SLOTS * std::max(t.K, 1);
  t.cnt->dev.reserve(words);
  if (clear) fill32(t.cnt->dev.p, 0, 2 * words, s);
}
static void fold_on_host(Counts &c, const long long *copies) {
  c.host.assign(c.K, 0);
  for (int sl = 0; sl < c.slots; sl++)
    for (int k = 0; k < c.K; k++) c.host[k] += copies[(size_t)sl * c.K + k];
  c.ready = true;
}
static void zero_counts(Table &t) {  // a table without rules
  t.cnt = std::make_shared<Counts>();
  t.cnt->K = t.K;
  t.cnt->host.assign(t.K, 0);
  t.cnt->ready = true;
}
void ensure_counts(Counts &c, hipStream_t s) {
  if (c.ready) return;
  std::vector<long long> h((size_t)c.K * c.slots);
  if (c.K && c.dev.p) {
    HIP_CHECK(hipMemcpyAsync(h.data(), c.dev.p, h.size() * sizeof(long long), hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipStreamSynchronize(s));
  }
  fold_on_host(c, h.data());
}
// A forward call over table t did per_rule multiply-adds per rule.  With macs != NULL the
// caller wants the number now; otherwise it is remembered and summed up by take_macs().
void note_macs(Metadata &m, Table &t, double per_rule, double *macs, hipStream_t s) {
  if (macs) {
    *macs = (double)t.total(s) * per_rule;
  } else if (t.cnt->ready) {
    m.macs_settled += (double)t.cnt->total() * per_rule;
  } else {
    m.pending_macs.emplace_back(t.cnt, per_rule);
  }
}
// Sum of the deferred multiply-add counts since the last call.  Every rulebook whose counts
// are still on the device is copied once, through a pinned staging buffer so that the copies
// are asynchronous, with one synchronisation per staging buffer's worth (in practice one).
double take_macs(Metadata &m, hipStream_t s) {
  static thread_local long long *stage = nullptr;
  constexpr size_t STAGE = 32768;  // entries: about thirty 27-tap rulebooks with all their copies
  if (!stage) HIP_CHECK(hipHostMalloc(reinterpret_cast<void **>(&stage), STAGE * sizeof(long long), hipHostMallocDefault));
  std::vector<Counts *> batch;
  size_t used = 0;
  auto flush = [&]() {
    if (batch.empty()) return;
    HIP_CHECK(hipStreamSynchronize(s));
    size_t off = 0;
    for (Counts *c : batch) {
      fold_on_host(*c, stage + off);
      off += (size_t)c->K * c->slots;
    }
    batch.clear();
    used = 0;
  };
  for (auto &pm : m.pending_macs) {
    Counts &c = *pm.first;
    if (c.ready || std::find(batch.begin(), batch.end(), &c) != batch.end()) continue;
    const size_t words = (size_t)c.K * c.slots;
    if (!c.K || !c.dev.p || words > STAGE) {  // nothing on the device (or absurdly many taps): the slow way
      ensure_counts(c, s);
      continue;
    }
    if (used + words > STAGE) flush();
    HIP_CHECK(hipMemcpyAsync(stage + used, c.dev.p, words * sizeof(long long), hipMemcpyDeviceToHost, s));
    used += words;
    batch.push_back(&c);
  }
  flush();
  for (auto &pm : m.pending_macs) m.macs_settled += (double)pm.first->total() * pm.second;
  m.pending_macs.clear();
  double r = m.macs_settled;
  m.macs_settled = 0;
  return r;
}

Table &submanifold_rules(Metadata &m, const int64_t *spatial, const int64_t *filter, hipStream_t s) {
  SizeKey key = mk(m.dim, spatial, filter);
  auto it = m.subm.find(key);
  if (it != m.subm.end()) return it->second;
  Filt f = make_filt(m.dim, filter, nullptr, nullptr);
  m.builds++;
  Table t;
  t.K = f.K;
  auto lit = m.levels.find(mk(m.dim, spatial));
  if (lit == m.levels.end() || lit->second.n == 0) {
    // Metadata/Metadata.cpp:445: an unknown level is an empty one.
    t.n = 0;
    t.npad = 64;
    t.identity_rows = true;
    zero_counts(t);
    return m.subm.emplace(key, std::move(t)).first->second;
  }
  Level &L = lit->second;
  t.n = L.n;
  t.npad = L.npad;
  bool all3 = true;
  for (int d = 0; d < m.dim; d++) all3 = all3 && f.size[d] == 3;
  if (all3 && (m.dim == 2 || m.dim == 3) && t.n <= TINY_MAX && !L.dups) {
    start_counts(t, s, false);
    int key_bits = 0;
    const PatternKey pk = pattern_plan(t.n, t.K, key_bits);
    const int passes = (key_bits + RS1_BITS - 1) / RS1_BITS, width = (key_bits + passes - 1) / passes;
    t.spread = pk.window >= t.n;
    t.nbr.reserve((size_t)t.K * t.npad);
    t.rowmap.reserve(t.npad);
    t.gmask.reserve(ceil_div(t.n, 16));
    const unsigned long long *keys = L.identity_sched ? L.keys.p : position_keys(L, s);
    unsigned long long *counts = reinterpret_cast<unsigned long long *>(t.cnt->dev.p);
    const int count_words = COUNT_SLOTS * t.K;
#define TINY_LAUNCH(D, C, T)                                                                                           \
  k_subm_tiny<D, C><<<dim3(1), T, 0, s>>>(L.g, keys, L.sched_ptr(), (int)t.n, t.npad, pk, key_bits, width, t.nbr.p,     \
                                         t.rowmap.p, t.gmask.p, counts, count_words)
    const bool few = t.n <= TINY_COUNT_MAX;
    if (m.dim == 3 && few) TINY_LAUNCH(3, true, TINY_COUNT_MAX);
    else if (m.dim == 3) TINY_LAUNCH(3, false, TINY_MAX);
    else if (few) TINY_LAUNCH(2, true, TINY_COUNT_MAX);
    else TINY_LAUNCH(2, false, TINY_MAX);
#undef TINY_LAUNCH
    LAUNCH_CHECK();
    t.identity_rows = false;
    return m.subm.emplace(key, std::move(t)).first->second;
  }
  // the counters are cleared by the launch that clears the level's block table, when this call builds it
  start_counts(t, s, false);
  const int64_t count_words = 2 * (int64_t)COUNT_SLOTS * std::max(t.K, 1);
  if (!ensure_grid(m, L, s, t.cnt->dev.p, (int)count_words)) fill32(t.cnt->dev.p, 0, count_words, s);
  if (all3 && (m.dim == 2 || m.dim == 3) && t.n > 0) {
    int key_bits = 0;
    const PatternKey pk = pattern_plan(t.n, t.K, key_bits);
    reserve_pattern_buffers(m, t);
    unsigned *masks = reinterpret_cast<unsigned *>(m.f1.p);
    const int roww = S3_ROW_INTS(m.dim);
    m.rowtab.reserve((size_t)t.npad * roww);
    if (m.dim == 3)
      k_subm_rules_s3<3, false><<<dim3((unsigned)(8 * ceil_div(ceil_div(L.n, 64), 8))), 192, 0, s>>>(L.g, L.g.bits, L.skeys.p, L.n, L.npad, L.table.p,
                                                           L.gridp.p, L.urow_ptr(), m.rowtab.p,
                                                           (unsigned long long *)t.cnt->dev.p, pk, m.k0.p, m.v0.p, masks, L.dups);
    else
      k_subm_rules_s3<2, false><<<dim3((unsigned)(8 * ceil_div(ceil_div(L.n, 64), 8))), 192, 0, s>>>(L.g, L.g.bits, L.skeys.p, L.n, L.npad, L.table.p,
                                                           L.gridp.p, L.urow_ptr(), m.rowtab.p,
                                                           (unsigned long long *)t.cnt->dev.p, pk, m.k0.p, m.v0.p, masks, L.dups);
    LAUNCH_CHECK();
    finalize_table(m, t, L.sched_ptr(), s, true, m.rowtab.p, roww);
    return m.subm.emplace(key, std::move(t)).first->second;
  }
  t.nbr.reserve((size_t)f.K * t.npad);
  // one wavefront per slice of the first filter dimension when that divides the taps evenly
  const int parts = (m.dim >= 2 && f.size[0] <= 4) ? f.size[0] : 1;
  k_subm_rules<<<grid_for(L.n, 64), 64 * parts, f.K * sizeof(int), s>>>(
      L.g, f, L.coords.p, L.sched_ptr(), L.n, L.npad, L.table.p, L.gridp.p, L.urow_ptr(), t.nbr.p,
      (unsigned long long *)t.cnt->dev.p, parts, L.dups ? L.skeys.p : nullptr);
  LAUNCH_CHECK();
  finalize_table(m, t, L.sched_ptr(), s);
  return m.subm.emplace(key, std::move(t)).first->second;
}

// ---- strided rules ---------------------------------------------------------------------

// Candidate output sites of every input site (Metadata/RectangularRegions.h:109-119):
// per dimension j in [max(0, ceil((p-size+1)/stride)), min(out-1, floor(p/stride))].
// Slot e = t * M + m holds the key of the m-th candidate of the row at position t, or EMPTY.
__device__ inline bool candidate(const Geom &gi, const Filt &f, const int *p, int m, int *j) {
  for (int d = f.dim - 1; d >= 0; d--) {
    int md = m % f.m[d];
    m /= f.m[d];
    int num = p[d] - f.size[d] + 1;
    int lb = num <= 0 ? 0 : (num + f.stride[d] - 1) / f.stride[d];
    int ub = min(f.out_size[d] - 1, p[d] / f.stride[d]);
    j[d] = lb + md;
    if (j[d] > ub) return false;
  }
  return true;
}

// pos_keys (optional, dimensions up to 3): the site key of every schedule position; the site is
// then decoded from one coalesced read instead of gathered by row through the schedule.
// dup_keys (levels whose keys may repeat, else null): the positions' keys; only the last position of a
// run of equal keys is a site (see k_subm_rules), the others have no candidates.
__global__ void k_strided_candidates(Geom gi, Geom go, Filt f, const int *soa, const int *sched,
                                     const unsigned long long *pos_keys, int64_t n, int64_t npad,
                                     unsigned long long *keys, int *payload, const unsigned long long *dup_keys) {
  int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n * f.M) return;
  int64_t t = e / f.M;
  int m = (int)(e - t * f.M);
  int p[SCN_MAXD], j[SCN_MAXD];
  int b;
  if (pos_keys) {
    site_of_key(gi, pos_keys[t], p, b);
  } else {
    const int row = sched ? sched[t] : (int)t;
    for (int d = 0; d < f.dim; d++) p[d] = soa[d * npad + row];
    b = soa[f.dim * npad + row];
  }
  const bool shadowed = dup_keys && t + 1 < n && dup_keys[t + 1] == dup_keys[t];
  keys[e] = (!shadowed && candidate(gi, f, p, m, j)) ? site_key(go, j, b) : SCN_EMPTY_KEY;
  payload[e] = (int)e;
}

// The same candidates without the slots that hold none (filters larger than their stride: a site
// of a 3^3 / stride-2 filter has 3.4 of its 8 on average, and the sort behind this is what a
// strided rulebook costs).  One thread per site, CB sites per workgroup; the first launch
// (WRITE = false) counts each workgroup's candidates, the second adds up the counts in front of
// its own, numbers its sites' candidates with a prefix inside the workgroup and writes them in
// (site, candidate) order; *n_valid = their number, which stays on the device (the launches
// behind are sized for n * M and look it up).
constexpr int CB = 256;
template <bool WRITE>
__global__ __launch_bounds__(CB) void k_strided_compact(Geom gi, Geom go, Filt f, const int *soa, const int *sched,
                                                        const unsigned long long *pos_keys, int64_t n, int64_t npad,
                                                        const unsigned long long *dup_keys, int *block_counts,
                                                        unsigned long long *keys, int *payload, int *n_valid) {
  __shared__ int part[CB / 64], wave_n[CB / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t = (int64_t)blockIdx.x * CB + threadIdx.x;
  int p[SCN_MAXD], j[SCN_MAXD], lb[SCN_MAXD], cnt[SCN_MAXD];
  int b = 0, mine = 0;
  const bool site = t < n && !(dup_keys && t + 1 < n && dup_keys[t + 1] == dup_keys[t]);
  if (site) {
    if (pos_keys) {
      site_of_key(gi, pos_keys[t], p, b);
    } else {
      const int row = sched ? sched[t] : (int)t;
      for (int d = 0; d < f.dim; d++) p[d] = soa[d * npad + row];
      b = soa[f.dim * npad + row];
    }
    // candidate() per dimension, once: the first output coordinate and how many there are; a
    // site's candidates are the product of the dimensions' ranges
    mine = 1;
    for (int d = 0; d < f.dim; d++) {
      const int num = p[d] - f.size[d] + 1;
      lb[d] = num <= 0 ? 0 : (num + f.stride[d] - 1) / f.stride[d];
      const int ub = min(f.out_size[d] - 1, p[d] / f.stride[d]);
      cnt[d] = max(0, min(ub - lb[d] + 1, f.m[d]));
      mine *= cnt[d];
    }
  }
  int incl = mine;  // inclusive prefix over the wavefront
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  if (lane == 63) wave_n[wave] = incl;
  if constexpr (!WRITE) {
    __syncthreads();
    if (threadIdx.x == 0) {
      int total = 0;
      for (int w = 0; w < CB / 64; w++) total += wave_n[w];
      block_counts[blockIdx.x] = total;
    }
    return;
  }
  int before = 0;
  for (int i = threadIdx.x; i < (int)blockIdx.x; i += CB) before += block_counts[i];
#pragma unroll
  for (int o = 32; o; o >>= 1) before += __shfl_xor(before, o, 64);
  if (lane == 0) part[wave] = before;
  __syncthreads();
  int pos = incl - mine, all = 0;
  for (int w = 0; w < CB / 64; w++) {
    pos += part[w] + (w < wave ? wave_n[w] : 0);
    all += part[w] + wave_n[w];
  }
  if (site && mine)
    for (int m = 0; m < f.M; m++) {  // numbered as candidate() numbers them: the last dimension fastest
      bool ok = true;
      int rest = m;
      for (int d = f.dim - 1; d >= 0; d--) {
        const int md = rest % f.m[d];
        rest /= f.m[d];
        j[d] = lb[d] + md;
        ok = ok && md < cnt[d];
      }
      if (ok) {
        keys[pos] = site_key(go, j, b);
        payload[pos] = (int)(t * f.M + m);
        pos++;
      }
    }
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) *n_valid = all;
}

// head[p] = 1 where a new output site begins in the sorted candidate keys.  n_dev (optional): the
// number of keys when only the device knows it; n is then the bound the launch is sized for.
__global__ void k_strided_heads(const unsigned long long *skeys, int64_t n, int *head, const int *n_dev) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p > n) return;
  const int64_t nv = n_dev ? *n_dev : n;
  if (p >= nv) {
    head[p] = 0;  // up to one element past the end, so that a scan of n + 1 ends with the total
    return;
  }
  const unsigned long long k = skeys[p];
  head[p] = (k != SCN_EMPTY_KEY && (p == 0 || k != skeys[p - 1])) ? 1 : 0;
}

// One thread per sorted candidate: output row = number of heads before it; the filter tap
// is the input site's offset inside the output's input box (Metadata/ConvolutionRules.h:19-31,
// Metadata/RectangularRegions.h:30-38,95-105).
__global__ void k_strided_emit(Geom gi, Filt f, const int *soa, const int *sched, const unsigned long long *pos_keys,
                               int64_t npad_in, const unsigned long long *skeys, const int *spayload, const int *head,
                               const int *head_scan, int64_t n_cand, int64_t npad_out, int *by_out,
                               int *by_in, int *out_soa, unsigned long long *out_keys,
                               unsigned long long *counts, const int *n_dev) {
  extern __shared__ int lcount[];  // per-block rule counts, flushed with one atomic per tap
  for (int k = threadIdx.x; k < f.K; k += blockDim.x) lcount[k] = 0;
  __syncthreads();
  if (n_dev) n_cand = *n_dev;
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  unsigned long long key = p < n_cand ? skeys[p] : SCN_EMPTY_KEY;
  if (key != SCN_EMPTY_KEY) {
    int e = spayload[p];
    int t = e / f.M, m = e - t * f.M;
    int row = sched ? sched[t] : t;
    int pc[SCN_MAXD], j[SCN_MAXD];
    int b;
    if (pos_keys) {
      site_of_key(gi, pos_keys[t], pc, b);
    } else {
      for (int d = 0; d < f.dim; d++) pc[d] = soa[d * npad_in + row];
      b = soa[f.dim * npad_in + row];
    }
    candidate(gi, f, pc, m, j);
    int k = 0;
    for (int d = 0; d < f.dim; d++) k = k * f.size[d] + (pc[d] - j[d] * f.stride[d]);
    int o = head_scan[p] + head[p] - 1;
    by_out[(int64_t)k * npad_out + o] = row;
    by_in[(int64_t)k * npad_in + t] = o;
    atomicAdd(&lcount[k], 1);
    if (head[p]) {
      for (int d = 0; d < f.dim; d++) out_soa[d * npad_out + o] = j[d];
      out_soa[f.dim * npad_out + o] = b;
      out_keys[o] = key;
    }
  }
  __syncthreads();
  unsigned long long *slot = counts + (size_t)(blockIdx.x & (COUNT_SLOTS - 1)) * f.K;
  for (int k = threadIdx.x; k < f.K; k += blockDim.x)
    if (lcount[k]) atomicAdd(&slot[k], (unsigned long long)lcount[k]);
}

// ---- filter = stride = 2 over exactly halving sizes (the U-Net's and most networks' downsampling) ----
// Every site has one output site, that of its coordinates halved, and the Morton key of that site
// ascends with the site's own key: in schedule order the inputs of an output site are neighbours
// (at most 2^dim of them), the output sites are the runs of equal parent keys, and nothing needs to
// be sorted.  Two launches make both tables, the output level and the keys of the pattern sort.
constexpr int HB = 512;  // positions per workgroup of the two kernels
// shift: the output level's key has one bit less per coordinate (sizes that halve exactly nearly
// always do), so the parent's key is the site's shifted down by dim bits and the tap, the site's
// offset inside its output site's 2^dim box, is the bits that fall out.
__device__ inline unsigned long long parent_key(const Geom &gi, const Geom &go, bool shift, unsigned long long key,
                                                int *tap) {
  if (shift) {
    *tap = (int)(key & ((1u << gi.dim) - 1u));
    return key >> gi.dim;
  }
  int p[SCN_MAXD], j[SCN_MAXD], b;
  site_of_key(gi, key, p, b);
  int k = 0;
  for (int d = 0; d < gi.dim; d++) {
    j[d] = p[d] >> 1;
    k = 2 * k + (p[d] & 1);
  }
  *tap = k;
  return site_key(go, j, b);
}
// block_heads[w] = output sites that begin in workgroup w's HB positions.
// counts (optional, 16 x 64 zeroed words): the sizes of the levels that `levels` further halvings
// will make.  Two sites fall into the same site j halvings further down iff their output keys agree
// above the low dim * j bits (a Morton key drops one bit per coordinate per halving; the sample
// index sits above), so in ascending key order a position starts a new site on every level up to
// (highest bit in which its output key differs from its predecessor's) / dim, and one pass counts
// the sites of all levels: counts[j], j = 0 .. levels, in one of 16 copies that the host adds up
// (thousands of workgroups adding to the same few addresses take longer than the rest of the
// kernel).  The whole chain of levels then costs one read-back instead of one per level.
// zero: words cleared for the launch behind this one.
__global__ __launch_bounds__(HB) void k_halve_heads(Geom gi, Geom go, bool shift, const unsigned long long *keys,
                                                    int64_t n, int levels, int *block_heads, int *counts,
                                                    uint32_t *zero, int zero_words) {
  __shared__ int hist[64];
  __shared__ int total;
  for (int i = blockIdx.x * HB + threadIdx.x; i < zero_words; i += gridDim.x * HB) zero[i] = 0u;
  if (threadIdx.x < 64) hist[threadIdx.x] = 0;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  const int64_t p = (int64_t)blockIdx.x * HB + threadIdx.x;
  int top = -1;  // a new site on levels 0 .. top
  if (p < n) {
    int tap;
    const unsigned long long ck = parent_key(gi, go, shift, keys[p], &tap);
    const unsigned long long d = p ? ck ^ parent_key(gi, go, shift, keys[p - 1], &tap) : ~0ull;
    if (d) top = p ? min(levels, (63 - __clzll((long long)d)) / gi.dim) : levels;
  }
  const unsigned long long heads = __ballot(top >= 0);
  if ((threadIdx.x & 63) == 0 && heads) atomicAdd(&total, __popcll(heads));
  if (counts)
    for (int l = 0; l <= levels; l++) {
      const unsigned long long bl = __ballot(top >= l);
      if ((threadIdx.x & 63) == 0 && bl) atomicAdd(&hist[l], __popcll(bl));
    }
  __syncthreads();
  if (threadIdx.x == 0) block_heads[blockIdx.x] = total;
  if (counts && threadIdx.x <= levels && hist[threadIdx.x])
    atomicAdd(&counts[(blockIdx.x & 15) * 64 + threadIdx.x], hist[threadIdx.x]);
}
// One thread per input position t: its output row o is the number of output sites that begin at or
// before t, less one (workgroups before this one: block_heads; inside: ballots).  It writes its own
// rule into by_out and as (tap, output row) for the fine-side table; the first position of an output site
// looks at the up to 2^dim - 1 positions behind it for the site's tap mask, writes -1 into the
// absent taps of by_out, the site's coordinates and key, and its pattern-sort key
// (Metadata/ConvolutionRules.h:19-31, Metadata/RectangularRegions.h:30-38,95-105 for this filter).
__global__ __launch_bounds__(HB) void k_halve_emit(Geom gi, Geom go, bool shift, const unsigned long long *keys, const int *sched,
                                                   int64_t n, int64_t npad_in, int64_t npad_out, const int *block_heads,
                                                   int *by_out, int *in_tap, int *in_row, int *out_soa, unsigned long long *out_keys,
                                                   unsigned long long *counts, PatternKey pk, unsigned long long *pkeys,
                                                   int *pidx, unsigned *pmasks, bool dups) {
  const int K = 1 << gi.dim;
  __shared__ int red[HB / 64], wave_heads[HB / 64], lcount[8];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int before = 0;
  for (int i = threadIdx.x; i < (int)blockIdx.x; i += HB) before += block_heads[i];
#pragma unroll
  for (int o = 32; o; o >>= 1) before += __shfl_xor(before, o, 64);
  if (threadIdx.x < 8) lcount[threadIdx.x] = 0;
  const int64_t p = (int64_t)blockIdx.x * HB + threadIdx.x;
  const bool live = p < n;
  int tap = -1;
  unsigned long long ck = 0;
  bool head = false;
  if (live) {
    ck = parent_key(gi, go, shift, keys[p], &tap);
    int t2;
    head = p == 0 || ck != parent_key(gi, go, shift, keys[p - 1], &t2);
  }
  const unsigned long long heads = __ballot(head);
  if (lane == 0) {
    red[wave] = before;
    wave_heads[wave] = __popcll(heads);
  }
  __syncthreads();
  int o = 0;
  for (int w = 0; w < HB / 64; w++) o += red[w] + (w < wave ? wave_heads[w] : 0);
  o += __popcll(heads & (~0ull >> (63 - lane))) - 1;  // heads at or before this lane, less one
  // dups (a level whose keys may repeat): only the last position of a run of equal keys is a site
  // (see k_subm_rules); the others have no rule, but may be where an output site's run begins
  const bool site = live && !(dups && p + 1 < n && keys[p + 1] == keys[p]);
  if (!site) tap = -1;
  if (live) {
    const int row = sched ? sched[p] : (int)p;
    in_tap[p] = tap;
    in_row[p] = o;
    if (site) by_out[(int64_t)tap * npad_out + o] = row;
    if (head) {
      unsigned mask = site ? 1u << tap : 0u;
      for (int i = 1; (dups || i < K) && p + i < n; i++) {
        int t2;
        const unsigned long long k2 = keys[p + i];
        if (parent_key(gi, go, shift, k2, &t2) != ck) break;
        if (!(dups && p + i + 1 < n && keys[p + i + 1] == k2)) mask |= 1u << t2;
      }
      int j[SCN_MAXD], b;
      site_of_key(go, ck, j, b);
      for (int k = 0; k < K; k++)
        if (!(mask >> k & 1u)) by_out[(int64_t)k * npad_out + o] = -1;
      for (int d = 0; d < gi.dim; d++) out_soa[d * npad_out + o] = j[d];
      out_soa[gi.dim * npad_out + o] = b;
      out_keys[o] = ck;
      pkeys[o] = pattern_key(pk, o, mask);
      pidx[o] = o;
      pmasks[o] = mask;
    }
  }
  for (int k = 0; k < K; k++) {
    const unsigned long long bk = __ballot(tap == k);
    if (lane == 0 && bk) atomicAdd(&lcount[k], __popcll(bk));
  }
  __syncthreads();
  unsigned long long *slot = counts + (size_t)(blockIdx.x & (COUNT_SLOTS - 1)) * K;
  if (threadIdx.x < K && lcount[threadIdx.x]) atomicAdd(&slot[threadIdx.x], (unsigned long long)lcount[threadIdx.x]);
}

// The same rulebook of a level of up to 1024 sites whose output size is known (a later link of a
// chain of halvings: the deep levels of a network), whole in one launch of one workgroup instead of
// four: k_halve_emit's work with the coarse-side table kept in LDS, the output sites' place in the
// pattern order by counting (as k_subm_tiny does) and the finished table, output rows and granule
// masks written from there.  zero / zero_words: every copy of the rule counters (copy 0 gets the counts).
constexpr int HALVE_SMALL = 1024;
__global__ __launch_bounds__(HALVE_SMALL) void k_halve_small(Geom gi, Geom go, bool shift, const unsigned long long *keys,
                                                             const int *sched, int n, int n_out, int64_t npad_out,
                                                             int *in_tap, int *in_row, int *out_soa,
                                                             unsigned long long *out_keys, PatternKey pk, int *nbr,
                                                             int *rowmap, unsigned *gmask, unsigned long long *counts,
                                                             int count_words) {
  const int K = 1 << gi.dim;
  __shared__ int lb[8][HALVE_SMALL];  // the coarse-side table before the sort: [tap][output site]
  __shared__ unsigned long long okey[HALVE_SMALL];
  __shared__ unsigned omask[HALVE_SMALL];
  __shared__ unsigned lg[HALVE_SMALL / 16];
  __shared__ int wave_heads[HALVE_SMALL / 64], lcount[8];
  const int p = threadIdx.x, lane = p & 63, wave = p >> 6;
  for (int i = p; i < 8 * HALVE_SMALL; i += HALVE_SMALL) (&lb[0][0])[i] = -1;
  for (int i = p; i < count_words; i += HALVE_SMALL) counts[i] = 0ull;
  if (p < 8) lcount[p] = 0;
  if (p < HALVE_SMALL / 16) lg[p] = 0u;
  const bool live = p < n;
  int tap = -1;
  unsigned long long ck = 0;
  bool head = false;
  if (live) {
    ck = parent_key(gi, go, shift, keys[p], &tap);
    int t2;
    head = p == 0 || ck != parent_key(gi, go, shift, keys[p - 1], &t2);
  }
  const unsigned long long heads = __ballot(head);
  if (lane == 0) wave_heads[wave] = __popcll(heads);
  __syncthreads();
  int o = 0;
  for (int w = 0; w < wave; w++) o += wave_heads[w];
  o += __popcll(heads & (~0ull >> (63 - lane))) - 1;  // heads at or before this lane, less one
  if (live) {
    in_tap[p] = tap;
    in_row[p] = o;
    lb[tap][o] = sched ? sched[p] : p;
    if (head) {
      unsigned mask = 1u << tap;
      for (int i = 1; i < K && p + i < n; i++) {
        int t2;
        if (parent_key(gi, go, shift, keys[p + i], &t2) != ck) break;
        mask |= 1u << t2;
      }
      int j[SCN_MAXD], b;
      site_of_key(go, ck, j, b);
      for (int d = 0; d < gi.dim; d++) out_soa[d * npad_out + o] = j[d];
      out_soa[gi.dim * npad_out + o] = b;
      out_keys[o] = ck;
      okey[o] = pattern_key(pk, o, mask);
      omask[o] = mask;
    }
  }
  for (int k = 0; k < K; k++) {
    const unsigned long long bk = __ballot(tap == k);
    if (lane == 0 && bk) atomicAdd(&lcount[k], __popcll(bk));
  }
  __syncthreads();
  // thread o < n_out: output site o goes to position P of the table
  if (p < n_out) {
    const unsigned long long mine = okey[p];
    int P = 0;
    for (int j = 0; j < n_out; j++) {
      const unsigned long long kj = okey[j];
      P += (kj < mine || (kj == mine && j < p)) ? 1 : 0;
    }
    for (int k = 0; k < K; k++) nbr[(int64_t)k * npad_out + P] = lb[k][p];
    rowmap[P] = p;
    atomicOr(&lg[P >> 4], omask[p]);
  }
  __syncthreads();
  if (p < (n_out + 15) / 16) gmask[p] = lg[p];
  if (p < K) counts[p] = (unsigned long long)lcount[p];
}

// ---- filters larger than their stride, small and middle levels: rules by lookup ----
// The sort of every (output site, input site) candidate is what such a rulebook costs on the
// general path.  Here the output sites are found first, as occupancy bits of their blocks of 64 keys
// in the block table that becomes the output level's site lookup (k_ob_mark); the blocks are listed
// (k_ob_list) and put in key order by counting, for each, the sites of the blocks with smaller keys,
// all pairs at once (k_ob_rank: a few thousand blocks at most); the sites are written in that order (k_ob_sites), which
// is the ascending key order the general path gives them; and the rules are looked up from the
// output side in the input level's table, as a submanifold rulebook's are.  The fine-side table is
// made the same way from the other side, when somebody asks for it (finish_by_in).
constexpr int OB_CAP = 65536;    // slots of the output level's block table on this path
constexpr int OB_MAX = 16384;    // blocks it may hold: above, the build falls back to the general path
constexpr int OB_PARTS = 32;     // k_ob_rank: pieces the blocks compared against are split into
constexpr int OB_MAX_M = 32;     // most candidates per input site
constexpr int OB_PROBES = 64;    // a probe sequence longer than this means a crowded table: fall back
constexpr int64_t OB_MAX_SITES = 400000;  // input sites above which the general path is taken right away
struct ObBlock {  // a block of the list
  unsigned long long key;
  int sites, slot;  // set bits of its mask; its slot in the table
};
// words: [0] blocks listed, [1] set when the path gives up, [2] output sites.
__global__ void k_ob_clear(BlockEntry *table, unsigned long long *gridp, int *words, uint32_t *zero, int zero_words) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b < OB_CAP) {
    table[b].key = SCN_EMPTY_KEY;
    table[b].mask = 0ull;
    table[b].base = 0;
  }
  if (b == 0) gridp[0] = OB_CAP - 1;
  if (b < 4) words[b] = 0;
  for (int i = b; i < zero_words; i += gridDim.x * blockDim.x) zero[i] = 0u;
}
// ORs `bits` into the entry of block bkey, claiming a slot for it when it has none: one atomic
// whose answer is waited for, one that is not.
__device__ inline void ob_insert(BlockEntry *table, unsigned long long bkey, unsigned long long bits, int *words) {
  unsigned long long b = hash64(bkey) & (OB_CAP - 1);
  for (int i = 0; i < OB_PROBES; i++) {
    const unsigned long long k = atomicCAS(&table[b].key, SCN_EMPTY_KEY, bkey);
    if (k == SCN_EMPTY_KEY || k == bkey) {
      atomicOr(&table[b].mask, bits);
      return;
    }
    b = (b + 1) & (OB_CAP - 1);
  }
  words[1] = 1;
}
// One thread per input position: its candidate output sites (Metadata/RectangularRegions.h:109-119),
// block by block.  The positions of a workgroup are neighbours in space and their candidates lie
// in a handful of blocks: they meet in a small table in LDS first, and the workgroup then
// inserts each of its blocks once (atomics on device memory are what this kernel would wait for).
constexpr int OB_LSLOTS = 256;
__global__ __launch_bounds__(TB) void k_ob_mark(Geom gi, Geom go, Filt f, const unsigned long long *pos_keys, int64_t n,
                                                bool dups, BlockEntry *table, int *words) {
  __shared__ unsigned long long lkey[OB_LSLOTS], lbits[OB_LSLOTS];
  for (int i = threadIdx.x; i < OB_LSLOTS; i += TB) {
    lkey[i] = SCN_EMPTY_KEY;
    lbits[i] = 0ull;
  }
  __syncthreads();
  auto put = [&](unsigned long long bkey, unsigned long long bits) {
    unsigned h = (unsigned)((bkey * 0x9E3779B97F4A7C15ull) >> 40) & (OB_LSLOTS - 1);
    for (int i = 0; i < OB_LSLOTS; i++) {
      const unsigned long long k = atomicCAS(&lkey[h], SCN_EMPTY_KEY, bkey);
      if (k == SCN_EMPTY_KEY || k == bkey) {
        atomicOr(&lbits[h], bits);
        return;
      }
      h = (h + 1) & (OB_LSLOTS - 1);
    }
    ob_insert(table, bkey, bits, words);  // more blocks than the small table holds (scattered points)
  };
  const int64_t t = (int64_t)blockIdx.x * TB + threadIdx.x;
  const bool stop = *reinterpret_cast<volatile int *>(words + 1) != 0;
  if (t < n && !stop && !(dups && t + 1 < n && pos_keys[t + 1] == pos_keys[t])) {
    int p[SCN_MAXD], j[SCN_MAXD], lb[SCN_MAXD], cnt[SCN_MAXD];
    int b;
    site_of_key(gi, pos_keys[t], p, b);
    // per dimension: the first output coordinate and how many there are (strides 1 and 2 without a division)
    for (int d = 0; d < 3; d++) {
      lb[d] = 0;
      cnt[d] = 1;
      if (d >= f.dim) continue;
      const int st = f.stride[d], num = p[d] - f.size[d] + 1;
      const int up = num <= 0 ? 0 : (st == 1 ? num : st == 2 ? (num + 1) >> 1 : (num + st - 1) / st);
      const int down = st == 1 ? p[d] : st == 2 ? p[d] >> 1 : p[d] / st;
      lb[d] = up;
      cnt[d] = max(0, min(min(f.out_size[d] - 1, down) - up + 1, f.m[d]));
    }
    // the candidates are the product of the ranges; their order does not matter here
    unsigned long long cur = SCN_EMPTY_KEY, bits = 0ull;
    for (int a0 = 0; a0 < cnt[0]; a0++)
      for (int a1 = 0; a1 < cnt[1]; a1++)
        for (int a2 = 0; a2 < cnt[2]; a2++) {
          j[0] = lb[0] + a0;
          j[1] = lb[1] + a1;
          j[2] = lb[2] + a2;
          const unsigned long long key = site_key(go, j, b);
          if ((key >> 6) != cur) {
            if (cur != SCN_EMPTY_KEY) put(cur, bits);
            cur = key >> 6;
            bits = 0ull;
          }
          bits |= 1ull << (key & 63);
        }
    if (cur != SCN_EMPTY_KEY) put(cur, bits);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < OB_LSLOTS; i += TB)
    if (lkey[i] != SCN_EMPTY_KEY) ob_insert(table, lkey[i], lbits[i], words);
}
// The blocks of the table, listed (in no order): one thread per slot, one atomic per workgroup.
__global__ __launch_bounds__(TB) void k_ob_list(const BlockEntry *table, ObBlock *list, int *words) {
  __shared__ int wave_n[TB / 64], wg_base;
  const int slot = blockIdx.x * TB + threadIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned long long key = table[slot].key;
  const bool live = key != SCN_EMPTY_KEY;
  const unsigned long long ballot = __ballot(live);
  if (lane == 0) wave_n[wave] = __popcll(ballot);
  __syncthreads();
  int before = 0, total = 0;
  for (int w = 0; w < TB / 64; w++) {
    before += w < wave ? wave_n[w] : 0;
    total += wave_n[w];
  }
  if (threadIdx.x == 0 && total) {
    wg_base = atomicAdd(&words[0], total);
    if (wg_base + total > OB_MAX) words[1] = 1;
  }
  __syncthreads();
  if (!live) return;
  const int i = wg_base + before + __popcll(ballot & ((1ull << lane) - 1ull));
  if (i < OB_MAX) {
    ObBlock e;
    e.key = key;
    e.sites = __popcll(table[slot].mask);
    e.slot = slot;
    list[i] = e;
  }
}
// base of every listed block = the sites of the listed blocks with smaller keys.  Workgroup
// (x, y): blocks 256 x .. of the list against piece y of it, a tile of 256 at a time through LDS:
// partial[y][r] = the sites of piece y's blocks in front of block r, which k_ob_sites adds up.
// words[2] = all sites.
__global__ __launch_bounds__(256) void k_ob_rank(const ObBlock *list, int *partial, int *words) {
  const int nb = words[0];
  if (words[1] || (int)blockIdx.x * 256 >= nb) return;
  __shared__ unsigned long long tkey[256];
  __shared__ int tpop[256];
  const int r = blockIdx.x * 256 + threadIdx.x;
  const unsigned long long key = r < nb ? list[r].key : 0ull;
  const int per = (nb + (int)gridDim.y - 1) / (int)gridDim.y;
  const int j0 = blockIdx.y * per, j1 = min(nb, j0 + per);
  int acc = 0, tot = 0;
  for (int base = j0; base < j1; base += 256) {
    const int j = base + threadIdx.x;
    __syncthreads();
    if (j < j1) {
      const ObBlock e = list[j];
      tkey[threadIdx.x] = e.key;
      tpop[threadIdx.x] = e.sites;
      tot += e.sites;
    }
    __syncthreads();
    const int cnt = min(256, j1 - base);
    int i = 0;
    for (; i + 4 <= cnt; i += 4) {  // four at a time: the reads of LDS overlap
      const unsigned long long k0 = tkey[i], k1 = tkey[i + 1], k2 = tkey[i + 2], k3 = tkey[i + 3];
      const int p0 = tpop[i], p1 = tpop[i + 1], p2 = tpop[i + 2], p3 = tpop[i + 3];
      acc += (k0 < key ? p0 : 0) + (k1 < key ? p1 : 0) + (k2 < key ? p2 : 0) + (k3 < key ? p3 : 0);
    }
    for (; i < cnt; i++) acc += tkey[i] < key ? tpop[i] : 0;
  }
  if (r < nb) partial[(size_t)blockIdx.y * OB_MAX + r] = acc;
  if (blockIdx.x == 0) {
    __shared__ int wg_tot;
    if (threadIdx.x == 0) wg_tot = 0;
    __syncthreads();
#pragma unroll
    for (int o = 32; o; o >>= 1) tot += __shfl_xor(tot, o, 64);
    if ((threadIdx.x & 63) == 0 && tot) atomicAdd(&wg_tot, tot);
    __syncthreads();
    if (threadIdx.x == 0 && wg_tot) atomicAdd(&words[2], wg_tot);
  }
}
// One wavefront per listed block, one lane per key of it: the block's base into the table and the
// output level's rows, in ascending key order.
__global__ __launch_bounds__(256) void k_ob_sites(Geom go, BlockEntry *table, const ObBlock *list, const int *partial, int nb,
                                                  int64_t npad, int *soa, unsigned long long *keys,
                                                  unsigned long long *skeys) {
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (r >= nb) return;
  int base = lane < OB_PARTS ? partial[(size_t)lane * OB_MAX + r] : 0;
#pragma unroll
  for (int o = 32; o; o >>= 1) base += __shfl_xor(base, o, 64);
  const ObBlock blk = list[r];
  BlockEntry *e = table + blk.slot;
  if (lane == 0) e->base = base;
  const unsigned long long mask = e->mask;
  if (!((mask >> lane) & 1ull)) return;
  const int row = base + __popcll(mask & ((1ull << lane) - 1ull));
  const unsigned long long key = (blk.key << 6) | (unsigned long long)lane;
  int c[SCN_MAXD], b;
  site_of_key(go, key, c, b);
  for (int d = 0; d < go.dim; d++) soa[d * npad + row] = c[d];
  soa[go.dim * npad + row] = b;
  keys[row] = key;
  skeys[row] = key;
}
// The fine-side table of such a rulebook: one thread per fine position, every tap k of its site p
// has the output site (p - k) / stride where that is whole and inside
// (Metadata/RectangularRegions.h:30-38,95-105), looked up in the coarse level's table.
__global__ void k_rules_from_fine(Geom gi, Geom go, Filt f, const unsigned long long *pos_keys, int64_t n, int64_t npad,
                                  bool dups, const BlockEntry *table, const unsigned long long *mask_p, int *nbr) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const unsigned long long mask = *mask_p;
  int p[SCN_MAXD], j[SCN_MAXD], tap[SCN_MAXD];
  int b;
  site_of_key(gi, pos_keys[t], p, b);
  const bool shadowed = dups && t + 1 < n && pos_keys[t + 1] == pos_keys[t];
  for (int d = 0; d < f.dim; d++) tap[d] = 0;
  unsigned long long last_bkey = SCN_EMPTY_KEY, last_bits = 0ull;
  int last_base = 0;
  for (int k = 0; k < f.K; k++) {
    bool ok = !shadowed;
    for (int d = 0; d < f.dim; d++) {
      const int num = p[d] - tap[d];
      j[d] = num / f.stride[d];
      ok = ok && num >= 0 && num % f.stride[d] == 0 && j[d] < f.out_size[d];
    }
    int r = -1;
    if (ok) {
      const unsigned long long key = site_key(go, j, b);
      if ((key >> 6) != last_bkey) {
        last_bkey = key >> 6;
        block_lookup(table, mask, last_bkey, last_bits, last_base);
      }
      const unsigned long long bit = 1ull << (key & 63);
      if (last_bits & bit) r = last_base + __popcll(last_bits & (bit - 1ull));
    }
    nbr[(int64_t)k * npad + t] = r;
    for (int d = f.dim - 1; d >= 0; d--) {  // next tap, last dimension fastest
      if (++tap[d] < f.size[d]) break;
      tap[d] = 0;
    }
  }
}

// false: more blocks than the path takes; nothing of it is left behind but LO's buffers.
static bool rules_by_lookup(Metadata &m, StridedRules &R, const Filt &f, const Geom &go, Level &LI, Level &LO, int batch,
                            hipStream_t s) {
  const int64_t n = LI.n;
  ensure_grid(m, LI, s);  // also leaves the positions' keys
  LO.table.reserve(OB_CAP);
  LO.gridp.reserve(2);
  m.ob_words.reserve(4);
  m.ob_list.reserve((size_t)OB_MAX * sizeof(ObBlock) / sizeof(int));
  ObBlock *list = reinterpret_cast<ObBlock *>(m.ob_list.p);
  m.ob_part.reserve((size_t)OB_PARTS * OB_MAX);
  start_counts(R.by_out, s, false);
  k_ob_clear<<<dim3(OB_CAP / TB), TB, 0, s>>>(LO.table.p, LO.gridp.p, m.ob_words.p, reinterpret_cast<uint32_t *>(R.by_out.cnt->dev.p),
                                              2 * COUNT_SLOTS * std::max(f.K, 1));
  LAUNCH_CHECK();
  k_ob_mark<<<grid_for(n), TB, 0, s>>>(LI.g, go, f, LI.skeys.p, n, LI.dups, LO.table.p, m.ob_words.p);
  LAUNCH_CHECK();
  k_ob_list<<<dim3(OB_CAP / TB), TB, 0, s>>>(LO.table.p, list, m.ob_words.p);
  LAUNCH_CHECK();
  k_ob_rank<<<dim3(OB_MAX / 256, OB_PARTS), 256, 0, s>>>(list, m.ob_part.p, m.ob_words.p);
  LAUNCH_CHECK();
  const int *w = fetch_words(m, m.ob_words.p, 4, s);
  if (w[1]) return false;
  const int nb = w[0];
  const int64_t n_out = w[2];
  alloc_level(LO, go, n_out, batch);
  LO.skeys.reserve(n_out + 1);
  if (nb) {
    k_ob_sites<<<dim3((unsigned)ceil_div(nb, 4)), 256, 0, s>>>(go, LO.table.p, list, m.ob_part.p, nb, LO.npad, LO.coords.p, LO.keys.p,
                                                             LO.skeys.p);
    LAUNCH_CHECK();
  }
  LO.grid_built = true;
  LO.skeys_ready = n_out > 0;
  LO.gen = ++m.level_gen;
  R.out_gen = LO.gen;
  R.by_out.n = n_out;
  R.by_out.npad = LO.npad;
  R.by_in.n = n;
  R.by_in.npad = LI.npad;
  R.by_in.cnt = R.by_out.cnt;  // both tables list the same rules
  R.by_in_lookup = true;
  if (n_out == 0) {
    R.by_out.identity_rows = true;
    return true;
  }
  unsigned long long *counts = reinterpret_cast<unsigned long long *>(R.by_out.cnt->dev.p);
  bool s3 = f.dim == 2 || f.dim == 3;
  for (int d = 0; d < f.dim; d++) s3 = s3 && f.size[d] == 3 && f.stride[d] == 2;
  if (s3) {
    int key_bits = 0;
    const PatternKey pk = pattern_plan(n_out, f.K, key_bits);
    reserve_pattern_buffers(m, R.by_out);
    unsigned *masks = reinterpret_cast<unsigned *>(m.f1.p);
    const int roww = S3_ROW_INTS(f.dim);
    m.rowtab.reserve((size_t)LO.npad * roww);
    const dim3 grid((unsigned)(8 * ceil_div(ceil_div(n_out, 64), 8)));
    if (f.dim == 3)
      k_subm_rules_s3<3, true><<<grid, 192, 0, s>>>(LI.g, go.bits, LO.skeys.p, n_out, LO.npad, LI.table.p, LI.gridp.p, LI.urow_ptr(),
                                                   m.rowtab.p, counts, pk, m.k0.p, m.v0.p, masks, false);
    else
      k_subm_rules_s3<2, true><<<grid, 192, 0, s>>>(LI.g, go.bits, LO.skeys.p, n_out, LO.npad, LI.table.p, LI.gridp.p, LI.urow_ptr(),
                                                   m.rowtab.p, counts, pk, m.k0.p, m.v0.p, masks, false);
    LAUNCH_CHECK();
    finalize_table(m, R.by_out, nullptr, s, true, m.rowtab.p, roww);
    return true;
  }
  R.by_out.nbr.reserve((size_t)f.K * LO.npad);
  const int parts = (f.dim >= 2 && f.size[0] <= 4) ? f.size[0] : 1;
  k_subm_rules<<<grid_for(n_out, 64), 64 * parts, f.K * sizeof(int), s>>>(LI.g, f, LO.coords.p, nullptr, n_out, LO.npad, LI.table.p,
                                                                        LI.gridp.p, LI.urow_ptr(), R.by_out.nbr.p, counts, parts,
                                                                        nullptr);
  LAUNCH_CHECK();
  finalize_table(m, R.by_out, nullptr, s);
  return true;
}
// A level about to be replaced: the rulebooks that would still look its sites up do it now.
static void settle_lookups(Metadata &m, const SizeKey &size, hipStream_t s) {
  for (auto &e : m.strided)
    if (e.second.by_in_lookup && e.second.out_size == size) finish_by_in(m, e.second, s);
}

StridedRules &strided_rules(Metadata &m, const int64_t *in_size, const int64_t *out_size,
                            const int64_t *filter, const int64_t *stride, hipStream_t s) {
  SizeKey key = mk(m.dim, in_size, filter, stride);
  auto it = m.strided.find(key);
  if (it != m.strided.end()) return it->second;
  Filt f = make_filt(m.dim, filter, stride, out_size);
  Geom go = make_geom(m.dim, out_size);
  m.builds++;
  StridedRules R;
  R.in_size = mk(m.dim, in_size);
  R.out_size = mk(m.dim, out_size);
  R.by_out.K = R.by_in.K = f.K;
  zero_counts(R.by_out);
  R.by_in.cnt = R.by_out.cnt;  // until rules are emitted below
  if (R.in_size == R.out_size) throw Error("strided rules: input and output spatial size coincide");

  auto lit = m.levels.find(R.in_size);
  int64_t n = lit == m.levels.end() ? 0 : lit->second.n;
  int batch = lit == m.levels.end() ? 0 : lit->second.batch;
  // Building a strided rulebook replaces the output level (Metadata/ConvolutionRules.h:68-70)
  // and whatever was cached for it.
  // Feature passes enqueued earlier may still be reading what is dropped here.
  if (m.levels.count(R.out_size)) {
    wait_for_consumers(m, s);
    settle_lookups(m, R.out_size, s);
  }
  for (auto i = m.subm.begin(); i != m.subm.end();)
    i = std::equal(R.out_size.begin(), R.out_size.end(), i->first.begin()) ? m.subm.erase(i) : std::next(i);
  Level &LO = m.levels[R.out_size];
  LO = Level();
  LO.identity_sched = true;
  if (n == 0) {
    alloc_level(LO, go, 0, batch);
    R.by_out.n = 0;
    R.by_out.npad = 64;
    R.by_in.n = 0;
    R.by_in.npad = 64;
    R.by_out.identity_rows = R.by_in.identity_rows = true;
    R.by_in_final = true;
    return m.strided.emplace(key, std::move(R)).first->second;
  }
  Level &LI = m.levels[R.in_size];
  int64_t nc = n * f.M;
  if (nc >= ((int64_t)1 << 31) - 64) throw Error("strided rules: too many candidate pairs for int32 indices");
  // Filter = stride = 2 in every dimension over exactly fitting sizes (the U-Net's and most
  // networks' downsampling): each site has one candidate, the Morton key of its coordinates
  // halved, which ascends with the site's own key, so the schedule order is already sorted.
  bool presorted = m.dim <= 3 && f.M == 1;
  for (int d = 0; d < m.dim; d++)
    presorted = presorted && filter[d] == 2 && stride[d] == 2 && in_size[d] == 2 * out_size[d];
  // The caller has to learn the new level's size: a read-back per rulebook, except along a chain
  // of exact halvings, whose sizes the first rulebook of the chain counts all at once
  // (k_halve_heads) and hands down from level to level.
  int chain = 0;  // further exact halvings of the output size, when this call has to count
  if (presorted && LI.halvings.empty()) {
    for (bool even = true; even && chain < 60 / m.dim - 1;) {
      for (int d = 0; d < m.dim; d++) even = even && (out_size[d] >> chain) % 2 == 0 && (out_size[d] >> chain) >= 2;
      if (even) chain++;
    }
    m.dflags.reserve(16 * 64);
  }
  const bool count = presorted && LI.halvings.empty();
  if (presorted && !count && n <= HALVE_SMALL && !LI.dups) {  // a small level of known output size: one launch
    const unsigned long long *keys = LI.identity_sched ? LI.keys.p : position_keys(LI, s);
    const int64_t n_out = LI.halvings[0];
    alloc_level(LO, go, n_out, batch);
    LO.halvings.assign(LI.halvings.begin() + 1, LI.halvings.end());
    R.by_out.n = n_out;
    R.by_out.npad = LO.npad;
    R.by_in.n = n;
    R.by_in.npad = LI.npad;
    R.by_out.nbr.reserve((size_t)f.K * LO.npad);
    R.by_out.rowmap.reserve(LO.npad);
    R.by_out.gmask.reserve(ceil_div(std::max<int64_t>(n_out, 1), 16));
    R.by_in_compact = true;
    R.in_tap.reserve(n);
    R.in_row.reserve(n);
    start_counts(R.by_out, s, false);
    int key_bits = 0;
    const PatternKey pk = pattern_plan(n_out, f.K, key_bits);
    R.by_out.spread = pk.window >= n_out;
    R.by_out.identity_rows = false;
    k_halve_small<<<dim3(1), HALVE_SMALL, 0, s>>>(LI.g, go, go.bits == LI.g.bits - 1, keys, LI.sched_ptr(), (int)n, (int)n_out,
                                                 LO.npad, R.in_tap.p, R.in_row.p, LO.coords.p, LO.keys.p, pk, R.by_out.nbr.p,
                                                 R.by_out.rowmap.p, R.by_out.gmask.p,
                                                 (unsigned long long *)R.by_out.cnt->dev.p, COUNT_SLOTS * f.K);
    LAUNCH_CHECK();
    R.by_in.cnt = R.by_out.cnt;  // both tables list the same rules
    return m.strided.emplace(key, std::move(R)).first->second;
  }
  if (presorted) {
    // positions' keys: the level's own when its rows are in schedule order (a level made here)
    const unsigned long long *keys = LI.identity_sched ? LI.keys.p : position_keys(LI, s);
    const int blocks = (int)ceil_div(n, HB);
    m.f0.reserve(blocks);
    start_counts(R.by_out, s, false);
    const int count_words = 2 * COUNT_SLOTS * f.K;
    if (count) fill32(m.dflags.p, 0, 16 * 64, s);
    const bool shift = go.bits == LI.g.bits - 1;
    k_halve_heads<<<dim3(blocks), HB, 0, s>>>(LI.g, go, shift, keys, n, chain, m.f0.p, count ? m.dflags.p : nullptr,
                                              reinterpret_cast<uint32_t *>(R.by_out.cnt->dev.p), count_words);
    LAUNCH_CHECK();
    if (count) {
      const int *c = fetch_words(m, m.dflags.p, 16 * 64, s);
      LI.halvings.assign(chain + 1, 0);
      for (int copy = 0; copy < 16; copy++)
        for (int l = 0; l <= chain; l++) LI.halvings[l] += c[copy * 64 + l];
    }
    const int64_t n_out = LI.halvings[0];
    alloc_level(LO, go, n_out, batch);
    LO.halvings.assign(LI.halvings.begin() + 1, LI.halvings.end());
    R.by_out.n = n_out;
    R.by_out.npad = LO.npad;
    R.by_in.n = n;
    R.by_in.npad = LI.npad;
    R.by_out.nbr.reserve((size_t)f.K * LO.npad);
    R.by_in_compact = true;
    R.in_tap.reserve(n);
    R.in_row.reserve(n);
    int key_bits = 0;
    const PatternKey pk = pattern_plan(n_out, f.K, key_bits);
    reserve_pattern_buffers(m, R.by_out);
    k_halve_emit<<<dim3(blocks), HB, 0, s>>>(LI.g, go, shift, keys, LI.sched_ptr(), n, LI.npad, LO.npad, m.f0.p, R.by_out.nbr.p,
                                             R.in_tap.p, R.in_row.p, LO.coords.p, LO.keys.p,
                                             (unsigned long long *)R.by_out.cnt->dev.p, pk, m.k0.p, m.v0.p,
                                             reinterpret_cast<unsigned *>(m.f1.p), LI.dups);
    LAUNCH_CHECK();
    R.by_in.cnt = R.by_out.cnt;  // both tables list the same rules
    finalize_table(m, R.by_out, nullptr, s, true);
    return m.strided.emplace(key, std::move(R)).first->second;
  }
  if (m.dim <= 3 && f.M > 1 && f.M <= OB_MAX_M && n <= OB_MAX_SITES) {
    R.filter.assign(filter, filter + m.dim);
    R.stride.assign(stride, stride + m.dim);
    if (rules_by_lookup(m, R, f, go, LI, LO, batch, s)) return m.strided.emplace(key, std::move(R)).first->second;
    LO = Level();  // too many blocks of output sites for that path (scattered points): the general one
    LO.identity_sched = true;
    zero_counts(R.by_out);
    R.by_in.cnt = R.by_out.cnt;
  }
  m.k0.reserve(nc);
  m.k1.reserve(nc);
  m.v0.reserve(nc);
  m.v1.reserve(nc);
  m.f0.reserve(nc + 1);
  m.s0.reserve(nc + 1);
  // a level with a schedule of its own (the input layer's): sites from the positions' keys
  const unsigned long long *pos_keys = (m.dim <= 3 && !LI.identity_sched) ? position_keys(LI, s) : nullptr;
  const unsigned long long *dup_keys = LI.dups ? position_keys(LI, s) : nullptr;
  const int *n_cand_dev = nullptr;
  if (f.M > 1 && nc > 32768 && nc <= ((int64_t)1 << 24)) {
    // only the slots that hold a candidate go into the sort; their number stays on the device
    const int blocks = (int)ceil_div(n, CB);
    m.f1.reserve(blocks);
    m.s1.reserve(1);
    k_strided_compact<false><<<dim3(blocks), CB, 0, s>>>(LI.g, go, f, LI.coords.p, LI.sched_ptr(), pos_keys, n, LI.npad,
                                                       dup_keys, m.f1.p, nullptr, nullptr, nullptr);
    LAUNCH_CHECK();
    k_strided_compact<true><<<dim3(blocks), CB, 0, s>>>(LI.g, go, f, LI.coords.p, LI.sched_ptr(), pos_keys, n, LI.npad,
                                                      dup_keys, m.f1.p, m.k0.p, m.v0.p, m.s1.p);
    LAUNCH_CHECK();
    n_cand_dev = m.s1.p;
    radix_sort_pairs(m, m.k0.p, m.k1.p, m.v0.p, m.v1.p, nc, std::min(64, key_bits(go, batch)), s, n_cand_dev);
  } else {
    k_strided_candidates<<<grid_for(nc), TB, 0, s>>>(LI.g, go, f, LI.coords.p, LI.sched_ptr(), pos_keys, n, LI.npad,
                                                     m.k0.p, m.v0.p, dup_keys);
    LAUNCH_CHECK();
    // one bit above the key bits keeps the EMPTY keys (all ones) behind every real key
    sort_pairs(m, m.k0.p, m.k1.p, m.v0.p, m.v1.p, nc, s, std::min(64, key_bits(go, batch) + 1));
  }
  k_strided_heads<<<grid_for(nc + 1), TB, 0, s>>>(m.k1.p, nc, m.f0.p, n_cand_dev);
  LAUNCH_CHECK();
  exclusive_scan(m, m.f0.p, m.s0.p, nc + 1, s);
  const int64_t n_out = fetch_words(m, m.s0.p + nc, 1, s)[0];
  alloc_level(LO, go, n_out, batch);
  R.by_out.n = n_out;
  R.by_out.npad = LO.npad;
  R.by_in.n = n;
  R.by_in.npad = LI.npad;
  R.by_out.nbr.reserve((size_t)f.K * LO.npad);
  R.by_in.nbr.reserve((size_t)f.K * LI.npad);
  start_counts(R.by_out, s, false);
  // both tables start empty and the counts at zero, in one launch
  fill3(R.by_out.nbr.p, 0xFFFFFFFFu, (int64_t)f.K * LO.npad, R.by_in.nbr.p, 0xFFFFFFFFu, (int64_t)f.K * LI.npad,
        R.by_out.cnt->dev.p, 0u, 2 * (int64_t)COUNT_SLOTS * std::max(f.K, 1), s);
  k_strided_emit<<<grid_for(nc), TB, f.K * sizeof(int), s>>>(LI.g, f, LI.coords.p, LI.sched_ptr(), pos_keys, LI.npad, m.k1.p, m.v1.p,
                                             m.f0.p, m.s0.p, nc, LO.npad, R.by_out.nbr.p, R.by_in.nbr.p,
                                             LO.coords.p, LO.keys.p, (unsigned long long *)R.by_out.cnt->dev.p, n_cand_dev);
  LAUNCH_CHECK();
  R.by_in.cnt = R.by_out.cnt;  // both tables list the same rules
  finalize_table(m, R.by_out, nullptr, s);
  return m.strided.emplace(key, std::move(R)).first->second;
}

// The fine-side table of a halving rulebook from its compact form: the positions in tap order
// (positions without a rule last), which gives a table whose rows have one tap each,
// inside windows of 1024 ITEMS consecutive schedule positions instead of a few
// ranges of the level, by one workgroup per window (block_sort, one 5-bit digit: no sort launches).
// A window's positions share their coarse rows (the 2^dim children of a site are neighbours in
// the schedule), so the taps' runs of a window, which one XCD works through at about the same
// time, find a coarse row that one of them fetched still in that XCD's L2; with an eighth of a
// million-site level per range every tap's run fetched its 4 MB of coarse rows again (counters:
// 268 MB read for 95 MB of operands).
template <int ITEMS>
__global__ __launch_bounds__(RS1_THREADS) void k_few_order(const int *in_tap, int64_t n, int *perm) {
  __shared__ BlockSort<ITEMS> sh;
  constexpr int WINDOW = RS1_THREADS * ITEMS;
  const int64_t base = (int64_t)blockIdx.x * WINDOW;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned long long key[ITEMS];
  int val[ITEMS];
  bool valid[ITEMS];
#pragma unroll
  for (int r = 0; r < ITEMS; r++) {
    const int i = wave * (ITEMS * 64) + r * 64 + lane;
    valid[r] = base + i < n;
    const int tap = valid[r] ? in_tap[base + i] : 0;
    key[r] = tap < 0 ? 16ull : (unsigned long long)tap;
    val[r] = i;
  }
  block_sort<ITEMS>(sh, key, val, valid, 5, 5);
  const int here = (int)min<int64_t>(WINDOW, n - base);
  for (int i = threadIdx.x; i < here; i += RS1_THREADS) perm[base + i] = (int)(base + sh.sval[i]);
}
// Position t of the sorted table is position perm[t] of the schedule: its one entry, -1 in the
// other taps, its row, and the granule masks (an OR over the 16 lanes of a granule).
__global__ void k_table_expand_few(const int *in_tap, const int *in_row, int K, int64_t n, int64_t npad, const int *perm,
                                   const int *base, int *nbr, int *rowmap, unsigned *gmask, unsigned char *few_tap,
                                   int *few_row) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  unsigned mk = 0;
  if (t < n) {
    const int src = perm[t];
    const int tap = in_tap[src], row = in_row[src];
    few_tap[t] = tap >= 0 ? (unsigned char)tap : (unsigned char)255;
    few_row[t] = tap >= 0 ? row : 0;
    for (int k = 0; k < K; k++) nbr[(int64_t)k * npad + t] = k == tap ? row : -1;
    mk = tap >= 0 ? 1u << tap : 0u;
    rowmap[t] = base ? base[src] : src;
  }
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) mk |= __shfl_xor(mk, o, 64);
  if ((threadIdx.x & 15) == 0 && t < n) gmask[t >> 4] = mk;
}

void finish_by_in(Metadata &m, StridedRules &r, hipStream_t s) {
  if (r.by_in_final) return;
  auto li = m.levels.find(r.in_size);
  if (li == m.levels.end()) throw Error("strided rules: the fine level is gone");
  m.builds++;
  Table &t = r.by_in;
  if (r.by_in_compact && t.n > 0) {
    m.v1.reserve(t.n);  // the order: position t of the table is position v1[t] of the schedule
    constexpr int FEW_ITEMS = 4;  // windows of 4096 positions (1024, 2048 and 8192 measured alike)
    const int window = RS1_THREADS * FEW_ITEMS;
    t.spread = window >= t.n;
    k_few_order<FEW_ITEMS><<<dim3((unsigned)ceil_div(t.n, window)), RS1_THREADS, 0, s>>>(r.in_tap.p, t.n, m.v1.p);
    LAUNCH_CHECK();
    t.nbr.reserve((size_t)t.K * t.npad);
    t.rowmap.reserve(t.npad);
    t.gmask.reserve(ceil_div(t.n, 16));
    t.few_tap.reserve(t.n);
    t.few_row.reserve(t.n);
    k_table_expand_few<<<grid_for(t.n), TB, 0, s>>>(r.in_tap.p, r.in_row.p, t.K, t.n, t.npad, m.v1.p,
                                                    li->second.sched_ptr(), t.nbr.p, t.rowmap.p, t.gmask.p, t.few_tap.p,
                                                    t.few_row.p);
    LAUNCH_CHECK();
    t.identity_rows = false;
    r.in_tap.release();
    r.in_row.release();
    r.by_in_compact = false;
    r.by_in_final = true;
    return;
  }
  if (r.by_in_lookup) {
    auto lo = m.levels.find(r.out_size);
    if (lo == m.levels.end() || lo->second.gen != r.out_gen)
      throw Error("strided rules: the coarse level was rebuilt before the fine-side table was made");
    Level &LI = li->second, &LO = lo->second;
    t.nbr.reserve((size_t)t.K * t.npad);
    if (t.n > 0) {
      ensure_grid(m, LI, s);  // the positions' keys (the table itself was needed to build the rulebook)
      const Filt f = make_filt(m.dim, r.filter.data(), r.stride.data(), r.out_size.data());
      k_rules_from_fine<<<grid_for(t.n), TB, 0, s>>>(LI.g, LO.g, f, LI.skeys.p, t.n, t.npad, LI.dups, LO.table.p, LO.gridp.p,
                                                   t.nbr.p);
      LAUNCH_CHECK();
    }
    r.by_in_lookup = false;
  }
  finalize_table(m, r.by_in, li->second.sched_ptr(), s);
  r.by_in_final = true;
}

// ---- identity table -----------------------------------------------------------------------

__global__ void k_identity_table(int64_t n, int64_t npad, int *nbr, unsigned *gmask) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < npad) nbr[t] = t < n ? (int)t : -1;
  if (t < (n + 15) / 16) gmask[t] = 1u;
}

// A 1x1 convolution (NetworkInNetwork, CPU/NetworkInNetwork.cpp:7-23) is the convolution
// over this table: one tap, position t reads row t and writes row t.
Table &identity_table(Metadata &m, int64_t rows, hipStream_t s) {
  auto it = m.ident.find(rows);
  if (it != m.ident.end()) return it->second;
  m.builds++;
  Table t;
  t.K = 1;
  t.n = rows;
  t.npad = round_up(std::max<int64_t>(rows, 1), 64);
  t.identity_rows = true;
  t.identity_few = true;
  t.cnt = std::make_shared<Counts>();
  t.cnt->K = 1;
  t.cnt->host.assign(1, rows);
  t.cnt->ready = true;
  if (rows > 0) {
    t.nbr.reserve(t.npad);
    t.gmask.reserve(ceil_div(rows, 16));
    k_identity_table<<<grid_for(t.npad), TB, 0, s>>>(rows, t.npad, t.nbr.p, t.gmask.p);
    LAUNCH_CHECK();
  }
  return m.ident.emplace(rows, std::move(t)).first->second;
}

// ---- pair-list export (ballot / prefix compaction) --------------------------------------

// Each wavefront counts its hits with a ballot, one lane reserves the range in the block's
// LDS counter, and lanes write at their prefix rank; blocks take their base from a scan of
// the per-block totals, so the list is ordered by schedule position and deterministic.
__global__ void k_tap_block_counts(const int *nbr, int64_t n, int *block_counts) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  bool hit = t < n && nbr[t] >= 0;
  unsigned long long bal = __ballot(hit);
  __shared__ int total;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) atomicAdd(&total, __popcll(bal));
  __syncthreads();
  if (threadIdx.x == 0) block_counts[blockIdx.x] = total;
}
__global__ void k_tap_compact(const int *nbr, const int *sched, int64_t n, const int *block_base,
                              bool swap, int *pairs) {
  int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int v = t < n ? nbr[t] : -1;
  bool hit = v >= 0;
  unsigned long long bal = __ballot(hit);
  int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __shared__ int wave_base[TB / 64];
  if (lane == 0) wave_base[wave] = __popcll(bal);
  __syncthreads();
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int w = 0; w < TB / 64; w++) {
      int c = wave_base[w];
      wave_base[w] = acc;
      acc += c;
    }
  }
  __syncthreads();
  if (hit) {
    int rank = __popcll(bal & ((1ull << lane) - 1ull));
    int64_t pos = (int64_t)block_base[blockIdx.x] + wave_base[wave] + rank;
    int row = sched ? sched[t] : (int)t;
    pairs[2 * pos + (swap ? 1 : 0)] = v;
    pairs[2 * pos + (swap ? 0 : 1)] = row;
  }
}
int64_t export_table_pairs(Metadata &m, Table &t, int k, bool swap, int *pairs, hipStream_t s) {
  const int *sched = t.rowmap_ptr();
  if (k < 0 || k >= t.K) throw Error("rule list index out of range");
  const int64_t count_k = t.counts(s)[k];
  if (t.n == 0 || count_k == 0) return 0;
  int64_t blocks = ceil_div(t.n, TB);
  m.f1.reserve(blocks + 1);
  m.s1.reserve(blocks + 1);
  const int *col = t.nbr.p + (int64_t)k * t.npad;
  k_tap_block_counts<<<dim3((unsigned)blocks), TB, 0, s>>>(col, t.n, m.f1.p);
  LAUNCH_CHECK();
  exclusive_scan(m, m.f1.p, m.s1.p, blocks, s);
  k_tap_compact<<<dim3((unsigned)blocks), TB, 0, s>>>(col, sched, t.n, m.s1.p, swap, pairs);
  LAUNCH_CHECK();
  return count_k;
}

// Sparse-to-dense lists: per sample, (row, row-major offset) (Metadata/ConvolutionRules.h:130-151).
__global__ void k_sample_hist(const int *soa_batch, int64_t n, int batch, unsigned long long *hist) {
  int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r < n) {
    int b = soa_batch[r];
    if (b >= 0 && b < batch) atomicAdd(&hist[b], 1ull);
  }
}
std::vector<int64_t> s2d_sizes(Metadata &m, const int64_t *spatial, hipStream_t s) {
  auto it = m.levels.find(mk(m.dim, spatial));
  if (it == m.levels.end()) return {};
  Level &L = it->second;
  std::vector<int64_t> out(L.batch, 0);
  if (L.n == 0 || L.batch == 0) return out;
  DevBuf<unsigned long long> hist;
  hist.reserve(L.batch);
  fill32(hist.p, 0, 2 * (int64_t)L.batch, s);
  k_sample_hist<<<grid_for(L.n), TB, 0, s>>>(L.coords.p + (int64_t)m.dim * L.npad, L.n, L.batch, hist.p);
  LAUNCH_CHECK();
  std::vector<unsigned long long> h(L.batch);
  HIP_CHECK(hipMemcpyAsync(h.data(), hist.p, L.batch * sizeof(long long), hipMemcpyDeviceToHost, s));
  HIP_CHECK(hipStreamSynchronize(s));
  out.assign(h.begin(), h.end());
  return out;
}
__global__ void k_s2d_flags(Geom g, const int *soa, int64_t n, int64_t npad, int sample, int *flag) {
  int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r < n) flag[r] = soa[g.dim * npad + r] == sample ? 1 : 0;
}
__global__ void k_s2d_pairs(Geom g, const int *soa, int64_t n, int64_t npad, const int *flag,
                            const int *scan, int *pairs) {
  int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= n || !flag[r]) return;
  int64_t off = 0;
  for (int d = 0; d < g.dim; d++) off = off * g.size[d] + soa[d * npad + r];
  pairs[2 * scan[r]] = (int)r;
  pairs[2 * scan[r] + 1] = (int)off;
}
int64_t export_s2d_pairs(Metadata &m, const int64_t *spatial, int sample, int *pairs, hipStream_t s) {
  auto it = m.levels.find(mk(m.dim, spatial));
  if (it == m.levels.end() || it->second.n == 0) return 0;
  Level &L = it->second;
  m.f1.reserve(L.n + 1);
  m.s1.reserve(L.n + 1);
  k_s2d_flags<<<grid_for(L.n), TB, 0, s>>>(L.g, L.coords.p, L.n, L.npad, sample, m.f1.p);
  LAUNCH_CHECK();
  exclusive_scan(m, m.f1.p, m.s1.p, L.n, s);
  k_s2d_pairs<<<grid_for(L.n), TB, 0, s>>>(L.g, L.coords.p, L.n, L.npad, m.f1.p, m.s1.p, pairs);
  LAUNCH_CHECK();
  return 0;
}

// Metadata/Metadata.cpp:351-411 (generateRuleBooks2s2 / 3s2): from the input level down, every
// level's 3^d submanifold table and the size-`size` stride-2 table to the next level, until an
// extent no longer halves (size 2: even and >= 2; size 3: odd and >= 3).
void generate_rulebooks(Metadata &m, int size, hipStream_t s) {
  if (size != 2 && size != 3) throw Error("rulebooks are precomputed for filter size 2 or 3 (stride 2)");
  if (m.input_size.empty()) throw Error("no input level to start from");
  int64_t in_s[SCN_MAXD], out_s[SCN_MAXD], f3[SCN_MAXD], fs[SCN_MAXD], st[SCN_MAXD];
  for (int d = 0; d < m.dim; d++) {
    in_s[d] = m.input_size[d];
    f3[d] = 3;
    fs[d] = size;
    st[d] = 2;
  }
  while (true) {
    submanifold_rules(m, in_s, f3, s);
    for (int d = 0; d < m.dim; d++) {
      if (size == 2 ? (in_s[d] < 2 || in_s[d] % 2 != 0) : (in_s[d] < 3 || in_s[d] % 2 != 1)) return;
      out_s[d] = size == 2 ? in_s[d] / 2 : (in_s[d] - 1) / 2;
    }
    strided_rules(m, in_s, out_s, fs, st, s);
    for (int d = 0; d < m.dim; d++) in_s[d] = out_s[d];
  }
}

}  // namespace scn
