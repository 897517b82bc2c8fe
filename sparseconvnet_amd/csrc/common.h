// Shared host/device helpers of libscn_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

#define SCN_MAXD 6
#define SCN_EMPTY_KEY 0xFFFFFFFFFFFFFFFFull

namespace scn {

struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

inline void hip_check(hipError_t e, const char *what, const char *file, int line) {
  if (e != hipSuccess) {
    char buf[512];
    snprintf(buf, sizeof buf, "%s failed: %s (%s:%d)", what, hipGetErrorString(e), file, line);
    throw Error(buf);
  }
}
#define HIP_CHECK(x) ::scn::hip_check((x), #x, __FILE__, __LINE__)
#define LAUNCH_CHECK() ::scn::hip_check(hipGetLastError(), "kernel launch", __FILE__, __LINE__)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// Device memory for the library's own buffers comes from a process-wide cache: blocks freed
// by one metadata object are handed to the next instead of going back to the driver, so a
// steady stream of scenes performs no hipMalloc / hipFree (each of which stalls the host,
// and hipFree the whole device).  Blocks are reused in the order work is enqueued.  The
// library enqueues on two streams, the caller's (convolutions and the other feature passes)
// and its own build stream (rulebook construction, see api.hip), so there are two caches and
// a block never moves from one to the other: whatever a thread allocates while it builds
// rulebooks (pool_scope() == POOL_BUILD) comes from and returns to the build cache.  An idle
// block remembers the stream of the call that returned it; a call on another stream that takes
// it first waits for that stream (callers may drive different handles from different streams;
// one handle is driven from one stream at a time).  A request takes the smallest idle block
// that fits if that wastes at most half of the request.
enum { POOL_COMPUTE = 0, POOL_BUILD = 1 };
int &pool_scope();  // the calling thread's current cache
void pool_set_stream(int pool, hipStream_t s);  // the stream the calling thread enqueues on for that cache
void *pool_alloc(size_t bytes, int pool);
void pool_free(void *p, size_t bytes, int pool);

// Owning device buffer.  Grows by reallocation (contents discarded).
template <class T> struct DevBuf {
  T *p = nullptr;
  size_t cap = 0;  // elements
  int pool = POOL_COMPUTE;  // the cache the block came from
  DevBuf() = default;
  DevBuf(const DevBuf &) = delete;
  DevBuf &operator=(const DevBuf &) = delete;
  DevBuf(DevBuf &&o) noexcept : p(o.p), cap(o.cap), pool(o.pool) { o.p = nullptr; o.cap = 0; }
  DevBuf &operator=(DevBuf &&o) noexcept {
    if (this != &o) {
      release();
      p = o.p;
      cap = o.cap;
      pool = o.pool;
      o.p = nullptr;
      o.cap = 0;
    }
    return *this;
  }
  ~DevBuf() { release(); }
  void release() {
    if (p) pool_free(p, cap * sizeof(T), pool);
    p = nullptr;
    cap = 0;
  }
  void reserve(size_t n) {
    if (n <= cap) return;
    release();
    pool = pool_scope();
    p = static_cast<T *>(pool_alloc(n * sizeof(T), pool));
    cap = n;
  }
  size_t bytes() const { return cap * sizeof(T); }
};

// Geometry of one level (one spatial size) and the packing of (sample, coordinates) into
// a 64-bit site key.  dim <= 3: Morton interleave of `bits` bits per coordinate with the
// sample index above, so ascending keys walk each sample along a Z-order curve; dim >= 4:
// row-major linear index.  Either way the key is a bijection on valid sites.
struct Geom {
  int dim;
  int bits;       // Morton bits per coordinate (dim <= 3)
  int64_t size[SCN_MAXD];
  int64_t vol;    // product of sizes (dim >= 4)
  int64_t max_batch;  // exclusive bound on the sample index that still fits the key
};

__host__ __device__ inline uint64_t spread2(uint64_t v) {  // 32 bits -> every 2nd bit
  v &= 0xFFFFFFFFull;
  v = (v | (v << 16)) & 0x0000FFFF0000FFFFull;
  v = (v | (v << 8)) & 0x00FF00FF00FF00FFull;
  v = (v | (v << 4)) & 0x0F0F0F0F0F0F0F0Full;
  v = (v | (v << 2)) & 0x3333333333333333ull;
  v = (v | (v << 1)) & 0x5555555555555555ull;
  return v;
}
__host__ __device__ inline uint64_t spread3(uint64_t v) {  // 21 bits -> every 3rd bit
  v &= 0x1FFFFFull;
  v = (v | (v << 32)) & 0x001F00000000FFFFull;
  v = (v | (v << 16)) & 0x001F0000FF0000FFull;
  v = (v | (v << 8)) & 0x100F00F00F00F00Full;
  v = (v | (v << 4)) & 0x10C30C30C30C30C3ull;
  v = (v | (v << 2)) & 0x1249249249249249ull;
  return v;
}

__host__ __device__ inline uint32_t compact2(uint64_t v) {  // every 2nd bit -> 32 bits (inverse of spread2)
  v &= 0x5555555555555555ull;
  v = (v | (v >> 1)) & 0x3333333333333333ull;
  v = (v | (v >> 2)) & 0x0F0F0F0F0F0F0F0Full;
  v = (v | (v >> 4)) & 0x00FF00FF00FF00FFull;
  v = (v | (v >> 8)) & 0x0000FFFF0000FFFFull;
  v = (v | (v >> 16)) & 0x00000000FFFFFFFFull;
  return (uint32_t)v;
}
__host__ __device__ inline uint32_t compact3(uint64_t v) {  // every 3rd bit -> 21 bits (inverse of spread3)
  v &= 0x1249249249249249ull;
  v = (v | (v >> 2)) & 0x10C30C30C30C30C3ull;
  v = (v | (v >> 4)) & 0x100F00F00F00F00Full;
  v = (v | (v >> 8)) & 0x001F0000FF0000FFull;
  v = (v | (v >> 16)) & 0x001F00000000FFFFull;
  v = (v | (v >> 32)) & 0x00000000001FFFFFull;
  return (uint32_t)v;
}

// c: dim coordinates, all inside [0, size).  The last coordinate varies fastest.
__host__ __device__ inline uint64_t site_key(const Geom &g, const int *c, int batch) {
  switch (g.dim) {
  case 1:
    return ((uint64_t)batch << g.bits) | (uint64_t)c[0];
  case 2:
    return ((uint64_t)batch << (2 * g.bits)) | (spread2(c[0]) << 1) | spread2(c[1]);
  case 3:
    return ((uint64_t)batch << (3 * g.bits)) | (spread3(c[0]) << 2) | (spread3(c[1]) << 1) |
           spread3(c[2]);
  default: {
    uint64_t k = (uint64_t)batch;
    for (int d = 0; d < g.dim; d++) k = k * (uint64_t)g.size[d] + (uint64_t)c[d];
    return k;
  }
  }
}

// Slot hash of a block key: one multiplication, the upper half of the product (tables have at
// most 2^31 slots).  Block keys are Morton keys without their low six bits: neighbours differ in
// low bits, which the multiplication carries into every bit above.  (The 64-bit finaliser this
// replaces cost the 3^d rule kernel 4 x 26 of its 1000 vector instructions per wavefront.)
__device__ inline uint64_t hash64(uint64_t k) { return (k * 0x9E3779B97F4A7C15ull) >> 32; }

// Site lookup.  Sites of a level, sorted by key, are cut into blocks of 64 consecutive key
// values (key >> 6: a 4x4x4 cell in 3-D, 8x8 in 2-D).  A block is one 32-byte entry of a small
// open-addressing table: its key, the 64-bit occupancy mask of its sites and the rank of its
// first site in the sorted order.  Looking a site up is one probe of that table (it holds
// about N/16 entries for surfaces, so it stays in L2) plus a popcount:
// rank = base + popcount(mask below the site's bit).  The 27 neighbours of a site fall into
// at most 8 blocks, and consecutive taps usually share one.
struct __attribute__((aligned(32))) BlockEntry {
  unsigned long long key;   // block key = site key >> 6, or SCN_EMPTY_KEY
  unsigned long long mask;  // bit i set: site with key (key << 6 | i) is active
  int base;                 // rank of the block's first site among the level's distinct sites
  int pad[3];
};

// Slot of the block with key bkey, or -1.  The table is at most half full; the trip count is
// bounded by the table size all the same so that no wave can spin on a damaged table.
__device__ inline int64_t block_find(const BlockEntry *table, uint64_t mask, uint64_t bkey) {
  uint64_t b = hash64(bkey) & mask;
  for (uint64_t i = 0; i <= mask; i++) {
    const unsigned long long k = table[b].key;
    if (k == bkey) return (int64_t)b;
    if (k == SCN_EMPTY_KEY) return -1;
    b = (b + 1) & mask;
  }
  return -1;
}

// Coordinates and sample index back from a site key; dimensions 1 to 3 (above, keys are linear indices).
__host__ __device__ inline void site_of_key(const Geom &g, uint64_t key, int *c, int &batch) {
  const uint64_t low = (1ull << g.bits) - 1ull;
  if (g.dim == 1) {
    c[0] = (int)(key & low);
  } else if (g.dim == 2) {
    c[0] = (int)(compact2(key >> 1) & low);
    c[1] = (int)(compact2(key) & low);
  } else {
    c[0] = (int)(compact3(key >> 2) & low);
    c[1] = (int)(compact3(key >> 1) & low);
    c[2] = (int)(compact3(key) & low);
  }
  batch = (int)(key >> (g.dim * g.bits));
}

// Occupancy bits and first row of the block with key bkey (false: no such block).  A slot's key
// and bits come with one 16-byte load, the row only when the key matches.
__device__ inline bool block_lookup(const BlockEntry *table, uint64_t mask, uint64_t bkey, unsigned long long &bits,
                                    int &base) {
  uint64_t b = hash64(bkey) & mask;
  for (uint64_t i = 0; i <= mask; i++) {
    const ulonglong2 km = *reinterpret_cast<const ulonglong2 *>(&table[b]);
    if (km.x == bkey) {
      bits = km.y;
      base = table[b].base;
      return true;
    }
    if (km.x == SCN_EMPTY_KEY) break;
    b = (b + 1) & mask;
  }
  bits = 0ull;
  base = 0;
  return false;
}

}  // namespace scn
