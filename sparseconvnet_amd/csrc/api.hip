// extern "C" surface of libscn_hip.so (declared in include/scn_hip.h).
#include "../../include/scn_hip.h"

#include "metadata.h"

using namespace scn;

struct scn_metadata {
  Metadata m;
};
struct scn_params {
  FrozenParams p;
};

static thread_local std::string g_error;

// ---- block cache behind DevBuf (see common.h) -----------------------------------------------
#include <atomic>
#include <map>
#include <mutex>
#include <tuple>
#include <unordered_map>

namespace scn {
namespace {
std::mutex g_pool_mutex;
// An idle block remembers the stream its last user enqueued on: handed to a call that runs on
// another stream, that stream is first made to wait for everything the old one holds.
struct IdleBlock {
  void *p;
  hipStream_t last;
  bool known;  // false: freed outside any call, by an owner that did not say where it was last used
};
std::multimap<std::tuple<int, int, size_t>, IdleBlock> g_pool;  // (device, cache, bytes) -> idle blocks
std::unordered_map<void *, size_t> g_block_bytes;                // every block the cache has handed out or holds
int64_t g_idle_bytes = 0, g_live_bytes = 0, g_peak_bytes = 0, g_mallocs = 0;

int current_device() {
  int d = 0;
  (void)hipGetDevice(&d);
  return d;
}

// Size classes: multiples of an eighth of the next power of two (at most 12.5% slack).
size_t size_class(size_t bytes) {
  size_t p2 = 4096;
  while (p2 < bytes) p2 <<= 1;
  size_t step = p2 / 8;
  return (bytes + step - 1) / step * step;
}

// The streams the calling thread is enqueueing on right now, per cache (set by the entry
// points and by BuildScope); `known` is false outside any call.
struct ThreadStreams {
  hipStream_t s[2] = {nullptr, nullptr};
  bool known[2] = {false, false};
};
ThreadStreams &thread_streams() {
  static thread_local ThreadStreams t;
  return t;
}

// Orders `to` behind everything enqueued on `from` so far.  Streams the caller has destroyed
// since cannot be recorded on: then the whole device is waited for.
void order_streams(hipStream_t from, hipStream_t to) {
  if (from == to) return;
  hipEvent_t ev = nullptr;
  if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) == hipSuccess && hipEventRecord(ev, from) == hipSuccess &&
      hipStreamWaitEvent(to, ev, 0) == hipSuccess) {
    (void)hipEventDestroy(ev);
    return;
  }
  if (ev) (void)hipEventDestroy(ev);
  (void)hipGetLastError();
  (void)hipDeviceSynchronize();
}

void release_idle_locked() {
  for (auto &kv : g_pool) {
    g_block_bytes.erase(kv.second.p);
    (void)hipFree(kv.second.p);
  }
  g_pool.clear();
  g_idle_bytes = 0;
}
}  // namespace

int &pool_scope() {
  static thread_local int scope = POOL_COMPUTE;
  return scope;
}
void pool_set_stream(int pool, hipStream_t s) {
  thread_streams().s[pool] = s;
  thread_streams().known[pool] = true;
}

void *pool_alloc(size_t bytes, int pool) {
  const size_t cls = size_class(bytes ? bytes : 1);
  const int dev = current_device();
  {
    std::unique_lock<std::mutex> lock(g_pool_mutex);
    // the smallest idle block that fits, unless it would waste more than half of the request
    auto it = g_pool.lower_bound(std::make_tuple(dev, pool, cls));
    if (it != g_pool.end() && std::get<0>(it->first) == dev && std::get<1>(it->first) == pool &&
        std::get<2>(it->first) <= cls + cls / 2) {
      const IdleBlock b = it->second;
      const size_t got = std::get<2>(it->first);
      g_pool.erase(it);
      g_idle_bytes -= (int64_t)got;
      g_live_bytes += (int64_t)got;
      lock.unlock();
      const ThreadStreams &t = thread_streams();
      if (!b.known) (void)hipDeviceSynchronize();
      else if (t.known[pool] && t.s[pool] != b.last) order_streams(b.last, t.s[pool]);
      return b.p;
    }
  }
  void *p = nullptr;
  hipError_t e = hipMalloc(&p, cls);
  if (e != hipSuccess) {
    // give idle blocks back to the driver and try once more
    (void)hipGetLastError();
    (void)hipDeviceSynchronize();
    {
      std::lock_guard<std::mutex> lock(g_pool_mutex);
      release_idle_locked();
    }
    HIP_CHECK(hipMalloc(&p, cls));
  }
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  g_block_bytes[p] = cls;
  g_live_bytes += (int64_t)cls;
  g_mallocs++;
  g_peak_bytes = std::max(g_peak_bytes, g_live_bytes + g_idle_bytes);
  return p;
}

void pool_free(void *p, size_t bytes, int pool) {
  if (!p) return;
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  hipPointerAttribute_t attr;
  int dev = hipPointerGetAttributes(&attr, p) == hipSuccess ? attr.device : current_device();
  auto it = g_block_bytes.find(p);
  const size_t got = it != g_block_bytes.end() ? it->second : size_class(bytes ? bytes : 1);
  g_live_bytes -= (int64_t)got;
  g_idle_bytes += (int64_t)got;
  g_pool.emplace(std::make_tuple(dev, pool, got), IdleBlock{p, thread_streams().s[pool], thread_streams().known[pool]});
}
}  // namespace scn

template <class F> static int guarded(F f) {
  try {
    f();
    return 0;
  } catch (const std::exception &e) {
    g_error = e.what();
    return 1;
  } catch (...) {
    g_error = "unknown failure";
    return 1;
  }
}

static Metadata &md(scn_metadata *h) {
  if (!h) throw Error("null metadata handle");
  return h->m;
}
// The stream argument of an entry point; whatever the call takes from or returns to the block
// cache is accounted to it.
static hipStream_t st(void *s) {
  pool_set_stream(POOL_COMPUTE, (hipStream_t)s);
  return (hipStream_t)s;
}

// ---- two streams -------------------------------------------------------------------------------
// Rulebooks depend on coordinates only, never on features.  They are built on a stream of the
// library's own (one per device, default priority), so that the many small kernels and the few
// host round trips of a construction run beside the convolutions already enqueued on the
// caller's stream instead of between them: the host gets ahead of the GPU, and a new scene's
// forward pass costs little more than its convolutions.  Ordering:
//   * a construction that reads the caller's data (the input layer's coordinates) first makes
//     the build stream wait for the caller's stream;
//   * behind every construction an event is recorded; every feature pass (and everything else
//     that reads rulebooks on the caller's stream) first makes its stream wait for the latest one;
//   * before a construction drops or overwrites something a feature pass may be reading, and
//     before a handle is destroyed, the build stream waits for the caller's stream.
// scn_set_build_stream(0), or SCN_BUILD_STREAM=0 in the environment, builds on the caller's
// stream as a single-stream library would.
static std::atomic<int> g_build_stream{-1};  // -1: not decided yet (environment), 0 / 1
static bool use_build_stream() {
  int v = g_build_stream.load();
  if (v < 0) {
    const char *e = getenv("SCN_BUILD_STREAM");
    v = (e && e[0] == '0') ? 0 : 1;
    g_build_stream.store(v);
  }
  return v != 0;
}
static hipStream_t device_build_stream() {
  static std::mutex mu;
  static std::map<int, hipStream_t> streams;
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  auto it = streams.find(dev);
  if (it != streams.end()) return it->second;
  hipStream_t s;
  HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  streams[dev] = s;
  return s;
}

struct BuildScope {
  Metadata &m;
  hipStream_t caller, bs;
  uint64_t builds0;
  int pool0;
  bool force = false;  // record the event even if no construction was counted
  // reads_caller_data: the construction reads buffers the caller filled on its stream, or
  // writes buffers the caller will read there
  BuildScope(Metadata &m_, void *stream, bool reads_caller_data = false)
      : m(m_), caller(st(stream)), bs(use_build_stream() ? device_build_stream() : st(stream)),
        builds0(m_.builds), pool0(pool_scope()) {
    pool_scope() = POOL_BUILD;
    pool_set_stream(POOL_BUILD, bs);
    if (bs != caller && reads_caller_data) {
      hipEvent_t ev;
      HIP_CHECK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
      HIP_CHECK(hipEventRecord(ev, caller));
      HIP_CHECK(hipStreamWaitEvent(bs, ev, 0));
      HIP_CHECK(hipEventDestroy(ev));
    }
  }
  hipStream_t s() const { return bs; }
  ~BuildScope() {
    pool_scope() = pool0;
    if (bs == caller || (m.builds == builds0 && !force)) return;
    m.build_stream = bs;
    hipEvent_t &ev = m.ready[m.ready_next];
    m.ready_next = (m.ready_next + 1) % 8;
    if (!ev && hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
      ev = nullptr;
      (void)hipStreamSynchronize(bs);  // no event to hand out: fall back to waiting here
      m.last_ready = nullptr;
      return;
    }
    if (hipEventRecord(ev, bs) != hipSuccess) {
      (void)hipStreamSynchronize(bs);
      m.last_ready = nullptr;
      return;
    }
    m.last_ready = ev;
    m.consumer_waited = false;
  }
};

// Called by everything that reads rulebooks or levels on the caller's stream.
static void consume(Metadata &m, hipStream_t s) {
  if (m.last_ready && (!m.consumer_waited || !m.consumer_known || m.consumer != s))
    HIP_CHECK(hipStreamWaitEvent(s, m.last_ready, 0));
  m.consumer = s;
  m.consumer_known = true;
  m.consumer_waited = true;
}

// ---- pinned host blocks ------------------------------------------------------------------------
// hipHostMalloc / hipHostFree cost tens of microseconds each and every new handle needs a few
// pinned words: blocks go back to a process-wide list instead of to the driver.
namespace scn {
namespace {
std::mutex g_pinned_mutex;
std::multimap<size_t, void *> g_pinned_idle;
}  // namespace
void *pinned_acquire(size_t bytes) {
  {
    std::lock_guard<std::mutex> lock(g_pinned_mutex);
    auto it = g_pinned_idle.find(bytes);
    if (it != g_pinned_idle.end()) {
      void *p = it->second;
      g_pinned_idle.erase(it);
      return p;
    }
  }
  void *p = nullptr;
  HIP_CHECK(hipHostMalloc(&p, bytes, hipHostMallocDefault));
  return p;
}
void pinned_release(void *p, size_t bytes) {
  if (!p) return;
  std::lock_guard<std::mutex> lock(g_pinned_mutex);
  g_pinned_idle.emplace(bytes, p);
}
}  // namespace scn

// ---- multiply-add counts of handles that are gone ---------------------------------------------
// A handle that is destroyed or cleared may still owe the caller the multiply-add counts of
// convolutions that did not ask for theirs (their rule counts are on the device).  Waiting for
// them there would stall the host on the whole forward pass each time a scene's metadata dies:
// instead the counts are copied to pinned memory behind the work already enqueued, an event
// marks the copy, and scn_take_released_macs folds whatever has been left behind.
namespace {
// The rule counts of up to 48 tables copied into one staging array by one launch: block b copies
// table b's words.  dst is pinned host memory (hipHostMalloc: device-accessible), so that a
// handle with forty tables costs the stream one short kernel instead of forty copies.
struct CountJobs {
  const long long *src[48];
  int off[48], words[48];
};
__global__ void k_gather_counts(CountJobs j, long long *dst) {
  const int b = blockIdx.x;
  for (int i = threadIdx.x; i < j.words[b]; i += blockDim.x) dst[j.off[b] + i] = j.src[b][i];
}
struct ReleasedMacs {
  hipEvent_t ev = nullptr;
  long long *stage = nullptr;
  size_t stage_bytes = 0;
  struct Item {
    size_t off;
    int K, slots;
    double per_rule;
  };
  std::vector<Item> items;
};
std::mutex g_released_mutex;
std::vector<ReleasedMacs> g_released;
double g_released_settled = 0;

void release_macs(Metadata &m) {
  double settled = m.macs_settled;
  m.macs_settled = 0;
  ReleasedMacs r;
  size_t words = 0;
  for (auto &pm : m.pending_macs) {
    Counts &c = *pm.first;
    if (c.ready || !c.K || !c.dev.p)
      settled += (c.ready ? (double)c.total() : 0.0) * pm.second;
    else
      words += (size_t)c.K * c.slots;
  }
  if (words) {
    try {
      // the stream the convolutions ran on; the rule counts are final before anything on it runs
      hipStream_t s = m.consumer_known ? m.consumer : nullptr;
      if (m.last_ready) HIP_CHECK(hipStreamWaitEvent(s, m.last_ready, 0));
      r.stage_bytes = round_up((int64_t)(words * sizeof(long long)), 1 << 16);
      r.stage = static_cast<long long *>(pinned_acquire(r.stage_bytes));
      size_t off = 0;
      CountJobs jobs{};
      int n_jobs = 0;
      auto flush = [&] {
        if (!n_jobs) return;
        k_gather_counts<<<dim3((unsigned)n_jobs), 64, 0, s>>>(jobs, r.stage);
        LAUNCH_CHECK();
        n_jobs = 0;
      };
      for (auto &pm : m.pending_macs) {
        Counts &c = *pm.first;
        if (c.ready || !c.K || !c.dev.p) continue;
        const size_t w = (size_t)c.K * c.slots;
        jobs.src[n_jobs] = c.dev.p, jobs.off[n_jobs] = (int)off, jobs.words[n_jobs] = (int)w;
        if (++n_jobs == 48) flush();
        r.items.push_back({off, c.K, c.slots, pm.second});
        off += w;
      }
      flush();
      HIP_CHECK(hipEventCreateWithFlags(&r.ev, hipEventDisableTiming));
      HIP_CHECK(hipEventRecord(r.ev, s));
    } catch (...) {  // a lost device: the counts are not worth an error in a destructor
      if (r.ev) (void)hipEventDestroy(r.ev);
      r.ev = nullptr;
      (void)hipGetLastError();
      (void)hipDeviceSynchronize();
      pinned_release(r.stage, r.stage_bytes);
      r = ReleasedMacs();
    }
  }
  m.pending_macs.clear();
  std::lock_guard<std::mutex> lock(g_released_mutex);
  g_released_settled += settled;
  if (r.ev) g_released.push_back(std::move(r));
}

double take_released_macs() {
  std::vector<ReleasedMacs> todo;
  double total;
  {
    std::lock_guard<std::mutex> lock(g_released_mutex);
    todo.swap(g_released);
    total = g_released_settled;
    g_released_settled = 0;
  }
  for (ReleasedMacs &r : todo) {
    if (hipEventSynchronize(r.ev) == hipSuccess) {
      for (const auto &it : r.items) {
        long long rules = 0;
        for (size_t i = 0; i < (size_t)it.K * it.slots; i++) rules += r.stage[it.off + i];
        total += (double)rules * it.per_rule;
      }
    } else {
      (void)hipGetLastError();
    }
    (void)hipEventDestroy(r.ev);
    pinned_release(r.stage, r.stage_bytes);
  }
  return total;
}
}  // namespace

static void retire(Metadata &m) {  // before the handle's buffers go back to the caches
  // the blocks were last used on the streams this handle was driven from
  if (m.consumer_known) pool_set_stream(POOL_COMPUTE, m.consumer);
  if (m.build_stream) pool_set_stream(POOL_BUILD, m.build_stream);
  if (m.build_stream) {
    try {
      wait_for_consumers(m, m.build_stream);
    } catch (...) {
      (void)hipDeviceSynchronize();
    }
  }
  for (hipEvent_t &e : m.ready) {
    if (e) (void)hipEventDestroy(e);
    e = nullptr;
  }
  m.last_ready = nullptr;
}

// Table lookups that may have to build: the construction runs on the build stream, then the
// caller's stream is made to wait for it.
static Table &subm_table(Metadata &m, const int64_t *spatial, const int64_t *filter, void *stream) {
  Table *t;
  {
    BuildScope b(m, stream);
    t = &submanifold_rules(m, spatial, filter, b.s());
  }
  consume(m, st(stream));
  return *t;
}
static StridedRules &strided_table(Metadata &m, const int64_t *in_size, const int64_t *out_size,
                                   const int64_t *filter, const int64_t *stride, void *stream) {
  StridedRules *r;
  {
    BuildScope b(m, stream);
    r = &strided_rules(m, in_size, out_size, filter, stride, b.s());
  }
  consume(m, st(stream));
  return *r;
}
// The same rulebook read from the fine side (transposed convolution, unpooling).
static StridedRules &strided_table_fine(Metadata &m, const int64_t *in_size, const int64_t *out_size,
                                        const int64_t *filter, const int64_t *stride, void *stream) {
  StridedRules *r;
  {
    BuildScope b(m, stream);
    r = &strided_rules(m, in_size, out_size, filter, stride, b.s());
    finish_by_in(m, *r, b.s());
  }
  consume(m, st(stream));
  return *r;
}
// Exports and other rarely used calls run wholly on the build stream, ordered against the
// caller's stream on both sides (they read and write the caller's buffers and use the
// constructions' scratch).
template <class F> static void on_build_stream(Metadata &m, void *stream, F f) {
  {
    BuildScope b(m, stream, true);
    b.force = true;
    f(b.s());
  }
  consume(m, st(stream));
}

// The three input routes: a construction that fails (coordinates outside the grid, a bad sample
// index, a full key) leaves the handle as it was before the call, ready for another attempt.
template <class F> static void build_input(Metadata &m, void *stream, F build) {
  try {
    BuildScope b(m, stream, true);
    build(b.s());
  } catch (...) {
    if (!m.input_size.empty()) m.levels.erase(m.input_size);
    m.input = InputRules();
    m.input_size.clear();
    throw;
  }
  // the construction's last kernels may still be reading the caller's buffers: whatever the
  // caller does with them next on its stream (free, reuse) is ordered behind them
  consume(m, st(stream));
}

static Level *find_level(Metadata &m, const int64_t *spatial) {
  auto it = m.levels.find(mk(m.dim, spatial));
  return it == m.levels.end() ? nullptr : &it->second;
}

extern "C" {

const char *scn_last_error(void) { return g_error.c_str(); }
int scn_rulebook_bits(void) { return 32; }

scn_metadata *scn_md_create(int dim) {
  if (dim < 1 || dim > SCN_MAXD) {
    g_error = "dimension must be 1..6";
    return nullptr;
  }
  try {
    scn_metadata *h = new scn_metadata();
    h->m.dim = dim;
    return h;
  } catch (const std::exception &e) {
    g_error = e.what();
    return nullptr;
  }
}
void scn_md_destroy(scn_metadata *h) {
  if (!h) return;
  release_macs(h->m);
  retire(h->m);
  const int scope = pool_scope();
  delete h;
  pool_scope() = scope;
}
int scn_md_clear(scn_metadata *h) {
  return guarded([&] {
    Metadata &m = md(h);
    release_macs(m);  // what the convolutions run so far still owe: scn_take_released_macs
    retire(m);
    m.levels.clear();
    m.subm.clear();
    m.strided.clear();
    m.ident.clear();
    m.input = InputRules();
    m.input_size.clear();
  });
}

int scn_set_build_stream(int enable) {
  const int before = use_build_stream() ? 1 : 0;
  g_build_stream.store(enable ? 1 : 0);
  return before;
}
int scn_md_set_bf16(scn_metadata *h, int enable) {
  return guarded([&] { md(h).bf16 = enable != 0; });
}
int scn_md_next_output_stride(scn_metadata *h, int64_t stride) {
  return guarded([&] {
    if (stride < 0) throw Error("output stride must not be negative");
    md(h).next_out_stride = stride;
  });
}
int scn_md_next_second_output(scn_metadata *h, float *out2, int64_t stride, const scn_bn_params *bn) {
  return guarded([&] {
    Metadata &m = md(h);
    if (!out2) {
      m.next_out2 = nullptr;
      return;
    }
    if (!bn || !bn->running_mean || !bn->running_var) throw Error("second output: needs a batch normalisation");
    if (stride <= 0) throw Error("second output: stride must be positive");
    m.next_out2 = out2;
    m.next_out2_stride = stride;
    m.next_out2_bn[0] = bn->running_mean;
    m.next_out2_bn[1] = bn->running_var;
    m.next_out2_bn[2] = bn->gamma;
    m.next_out2_bn[3] = bn->beta;
    m.next_out2_eps = bn->eps;
    m.next_out2_leak = bn->leakiness;
  });
}
const char *scn_md_last_conv_kernel(scn_metadata *h) { return h ? h->m.last_kernel.c_str() : ""; }
int scn_md_input_layer(scn_metadata *h, const int64_t *spatial, const int64_t *coords, int64_t n,
                       int ncols, int min_batch, int mode, void *stream, int64_t *n_active) {
  return guarded([&] {
    Metadata &m = md(h);
    if (n < 0) throw Error("negative point count");
    if (m.input.mode >= 0) throw Error("this metadata already has an input layer; call scn_md_clear first");
    build_input(m, stream, [&](hipStream_t s) { build_input_layer(m, spatial, CoordSrc{coords, 8}, n, ncols, min_batch, mode, s); });
    if (n_active) *n_active = m.input.n_out;
  });
}
int scn_md_input_layer_host(scn_metadata *h, const int64_t *spatial, const int64_t *host_coords, int64_t n,
                            int ncols, int min_batch, int mode, void *stream, int64_t *n_active) {
  return guarded([&] {
    Metadata &m = md(h);
    if (n < 0) throw Error("negative point count");
    if (m.input.mode >= 0) throw Error("this metadata already has an input layer; call scn_md_clear first");
    bool allow16 = true;
    for (int d = 0; d < m.dim; d++) allow16 = allow16 && spatial[d] <= 32767;
    try {
      build_input(m, stream, [&](hipStream_t s) {
        const CoordSrc src = stage_host_coords(m, host_coords, n * ncols, s, allow16);
        build_input_layer(m, spatial, src, n, ncols, min_batch, mode, s);
      });
    } catch (...) {
      (void)hipDeviceSynchronize();  // copies out of the pinned block may still be under way
      release_staging(m);
      throw;
    }
    release_staging(m);
    if (n_active) *n_active = m.input.n_out;
  });
}
int scn_md_input_batch(scn_metadata *h, const int64_t *spatial, const int64_t *coords,
                       const unsigned char *overwrite, int64_t n, int ncols, int min_batch, void *stream,
                       int64_t *n_active) {
  return guarded([&] {
    Metadata &m = md(h);
    if (n < 0) throw Error("negative point count");
    if (m.input.mode >= 0) throw Error("this metadata already has an input layer; call scn_md_clear first");
    build_input(m, stream, [&](hipStream_t s) {
      build_input_layer(m, spatial, CoordSrc{coords, 8}, n, ncols, min_batch, 5, s, 0, overwrite);  // `overwrite` is copied
    });
    if (n_active) *n_active = m.input.n_out;
  });
}
int scn_md_generate_rulebooks(scn_metadata *h, int size, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    BuildScope b(m, stream);
    generate_rulebooks(m, size, b.s());
  });
}
int scn_md_input_rules_header(scn_metadata *h, int32_t hdr[4]) {
  return guarded([&] {
    Metadata &m = md(h);
    if (m.input.mode < 0) throw Error("input layer rules have not been built");
    hdr[0] = m.input.user_mode;
    hdr[1] = input_max_active(m);
    hdr[2] = (int32_t)m.input.n_in;
    hdr[3] = (int32_t)m.input.n_out;
  });
}
int scn_md_bl_input_layer(scn_metadata *h, const int64_t *spatial, const int64_t *coords, int64_t batch,
                          int64_t length, int mode, void *stream, int64_t *n_active) {
  return guarded([&] {
    Metadata &m = md(h);
    if (batch < 0 || length < 0) throw Error("negative batch size or length");
    if (m.input.mode >= 0) throw Error("this metadata already has an input layer; call scn_md_clear first");
    if (batch * length == 0) length = 1, batch = 0;
    build_input(m, stream, [&](hipStream_t s) {
      build_input_layer(m, spatial, CoordSrc{coords, 8}, batch * length, m.dim, 0, mode, s, length);
    });
    if (n_active) *n_active = m.input.n_out;
  });
}
int scn_md_bl_rules_header(scn_metadata *h, int32_t hdr[5]) {
  return guarded([&] {
    Metadata &m = md(h);
    if (m.input.mode < 0 || m.input.bl_length == 0) throw Error("batch-by-length input rules have not been built");
    hdr[0] = m.input.user_mode;
    hdr[1] = input_max_active(m);
    hdr[2] = (int32_t)m.input.bl_batch;
    hdr[3] = (int32_t)m.input.bl_length;
    hdr[4] = (int32_t)m.input.n_out;
  });
}
int scn_md_input_rules(scn_metadata *h, int32_t *rows, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    on_build_stream(m, stream, [&](hipStream_t s) { export_input_rules(m, rows, s); });
  });
}
int scn_md_nactive(scn_metadata *h, const int64_t *spatial, int64_t *n_active) {
  return guarded([&] {
    Level *l = find_level(md(h), spatial);
    *n_active = l ? l->n : 0;
  });
}
int scn_md_batch_size(scn_metadata *h, const int64_t *spatial, int *batch) {
  return guarded([&] {
    Level *l = find_level(md(h), spatial);
    *batch = l ? l->batch : 0;
  });
}
int scn_md_spatial_locations(scn_metadata *h, const int64_t *spatial, int64_t *out, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    on_build_stream(m, stream, [&](hipStream_t s) { spatial_locations(m, spatial, out, s); });
  });
}
int scn_md_submanifold_rules(scn_metadata *h, const int64_t *spatial, const int64_t *filter, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    BuildScope b(m, stream);
    submanifold_rules(m, spatial, filter, b.s());
  });
}
int scn_md_strided_rules(scn_metadata *h, const int64_t *in_size, const int64_t *out_size,
                         const int64_t *filter, const int64_t *stride, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    BuildScope b(m, stream);
    strided_rules(m, in_size, out_size, filter, stride, b.s());
  });
}

int scn_rules_count(scn_metadata *h, int kind, const int64_t *a, const int64_t *b, const int64_t *c,
                    const int64_t *d, void *stream, int *count) {
  return guarded([&] {
    Metadata &m = md(h);
    if (kind == 0)
      *count = subm_table(m, a, b, stream).K;
    else if (kind == 1)
      *count = strided_table(m, a, b, c, d, stream).by_out.K;
    else if (kind == 2) {
      Level *l = find_level(m, a);
      *count = l ? l->batch : 0;
    } else
      throw Error("unknown rulebook kind");
  });
}
int scn_md_take_macs(scn_metadata *h, void *stream, double *macs) {
  return guarded([&] {
    Metadata &m = md(h);
    consume(m, st(stream));
    *macs = take_macs(m, st(stream));
  });
}
int scn_take_released_macs(double *macs) {
  return guarded([&] { *macs = take_released_macs(); });
}
int scn_release_cache(void) {
  return guarded([&] {
    HIP_CHECK(hipDeviceSynchronize());
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    release_idle_locked();
  });
}
int scn_cache_stats(int64_t *live_bytes, int64_t *idle_bytes, int64_t *peak_bytes, int64_t *device_allocations) {
  return guarded([&] {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    if (live_bytes) *live_bytes = g_live_bytes;
    if (idle_bytes) *idle_bytes = g_idle_bytes;
    if (peak_bytes) *peak_bytes = g_peak_bytes;
    if (device_allocations) *device_allocations = g_mallocs;
  });
}
int scn_sort_pairs(scn_metadata *h, const unsigned long long *keys_in, unsigned long long *keys_out, const int *values_in,
                   int *values_out, int64_t n, int end_bit, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    if (n < 0 || end_bit < 1 || end_bit > 64) throw Error("sort: n must not be negative, end_bit in 1..64");
    radix_sort_pairs(m, keys_in, keys_out, values_in, values_out, n, end_bit, static_cast<hipStream_t>(stream));
  });
}
int scn_rules_sizes(scn_metadata *h, int kind, const int64_t *a, const int64_t *b, const int64_t *c,
                    const int64_t *d, void *stream, int64_t *sizes) {
  return guarded([&] {
    Metadata &m = md(h);
    std::vector<int64_t> v;
    if (kind == 0) {
      v = subm_table(m, a, b, stream).counts(st(stream));
    } else if (kind == 1) {
      v = strided_table(m, a, b, c, d, stream).by_out.counts(st(stream));
    } else if (kind == 2)
      on_build_stream(m, stream, [&](hipStream_t s) { v = s2d_sizes(m, a, s); });
    else
      throw Error("unknown rulebook kind");
    for (size_t i = 0; i < v.size(); i++) sizes[i] = v[i];
  });
}
int scn_rules_export(scn_metadata *h, int kind, const int64_t *a, const int64_t *b, const int64_t *c,
                     const int64_t *d, int k, int32_t *pairs, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    if (kind == 0) {
      on_build_stream(m, stream, [&](hipStream_t s) {
        Table &t = submanifold_rules(m, a, b, s);
        export_table_pairs(m, t, k, false, pairs, s);
      });
    } else if (kind == 1) {
      on_build_stream(m, stream, [&](hipStream_t s) {
        StridedRules &r = strided_rules(m, a, b, c, d, s);
        export_table_pairs(m, r.by_out, k, false, pairs, s);
      });
    } else if (kind == 2) {
      on_build_stream(m, stream, [&](hipStream_t s) { export_s2d_pairs(m, a, k, pairs, s); });
    } else
      throw Error("unknown rulebook kind");
  });
}

int scn_input_layer_fwd(scn_metadata *h, const float *in, float *out, int planes, void *stream) {
  return guarded([&] {
    consume(md(h), st(stream));
    input_forward(md(h).input, in, out, planes, st(stream));
  });
}
int scn_output_layer_fwd(scn_metadata *h, const float *in, float *out, int planes, void *stream) {
  return guarded([&] {
    consume(md(h), st(stream));
    output_forward(md(h).input, in, out, planes, st(stream));
  });
}

static int64_t level_rows(Metadata &m, const int64_t *spatial) {
  Level *l = find_level(m, spatial);
  return l ? l->n : 0;
}
static void subm_conv(scn_metadata *h, const int64_t *spatial, const int64_t *filter, const float *in, float *out,
                      const float *weight, const float *bias, int n_in, int n_out, int groups, const BnArgs *pre,
                      const BnArgs *post, void *stream, double *macs) {
  Metadata &m = md(h);
  Table &t = subm_table(m, spatial, filter, stream);
  conv_forward(m, t, in, level_rows(m, spatial), out, weight, bias, n_in, n_out, groups, pre, post, st(stream));
  // CPU/Convolution.cpp:141: nRules * ip * op * groups per tap
  note_macs(m, t, (double)(n_in / groups) * (n_out / groups) * groups, macs, st(stream));
}
static void strided_conv(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *filter,
                         const int64_t *stride, const float *in, float *out, const float *weight,
                         const float *bias, int n_in, int n_out, int groups, const BnArgs *pre, const BnArgs *post,
                         void *stream, double *macs) {
  Metadata &m = md(h);
  StridedRules &r = strided_table(m, in_size, out_size, filter, stride, stream);
  conv_forward(m, r.by_out, in, level_rows(m, in_size), out, weight, bias, n_in, n_out, groups, pre, post,
               st(stream));
  note_macs(m, r.by_out, (double)(n_in / groups) * (n_out / groups) * groups, macs, st(stream));
}
static void deconv(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *filter,
                   const int64_t *stride, const float *in, float *out, const float *weight, const float *bias,
                   int n_in, int n_out, int groups, const BnArgs *pre, const BnArgs *post, void *stream,
                   double *macs) {
  Metadata &m = md(h);
  // CPU/Deconvolution.cpp:15-16: the rulebook of (out_size -> in_size), columns swapped.
  StridedRules &r = strided_table_fine(m, out_size, in_size, filter, stride, stream);
  conv_forward(m, r.by_in, in, level_rows(m, in_size), out, weight, bias, n_in, n_out, groups, pre, post,
               st(stream));
  note_macs(m, r.by_in, (double)(n_in / groups) * (n_out / groups) * groups, macs, st(stream));
}

int scn_subm_conv_fwd(scn_metadata *h, const int64_t *spatial, const int64_t *filter, const float *in,
                      float *out, const float *weight, const float *bias, int n_in, int n_out,
                      int groups, void *stream, double *macs) {
  return guarded([&] {
    subm_conv(h, spatial, filter, in, out, weight, bias, n_in, n_out, groups, nullptr, nullptr, stream, macs);
  });
}
int scn_subm_conv_fwd_noalloc(scn_metadata *h, const int64_t *spatial, const int64_t *filter, const float *in,
                              float *out, const float *weight, const float *bias, int n_in, int n_out,
                              void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    auto it = m.subm.find(mk(m.dim, spatial, filter));
    if (it == m.subm.end())
      throw Error("allocation-free convolution: build the rulebook first (scn_md_submanifold_rules)");
    Table &t = it->second;
    consume(m, st(stream));  // waits on an event that exists already; creates nothing
    struct Fixed {  // the kernels' scratch is the static array for the length of this call
      Metadata &m;
      Fixed(Metadata &m_) : m(m_) { m.fixed_scratch = noalloc_scratch(); }
      ~Fixed() { m.fixed_scratch = nullptr; }
    } fixed(m);
    conv_forward(m, t, in, level_rows(m, spatial), out, weight, bias, n_in, n_out, 1, nullptr, nullptr, st(stream));
    note_macs(m, t, (double)n_in * n_out, nullptr, st(stream));
  });
}
int scn_conv_fwd(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *filter,
                 const int64_t *stride, const float *in, float *out, const float *weight,
                 const float *bias, int n_in, int n_out, int groups, void *stream, double *macs) {
  return guarded([&] {
    strided_conv(h, in_size, out_size, filter, stride, in, out, weight, bias, n_in, n_out, groups, nullptr, nullptr,
                 stream, macs);
  });
}
int scn_deconv_fwd(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *filter,
                   const int64_t *stride, const float *in, float *out, const float *weight,
                   const float *bias, int n_in, int n_out, int groups, void *stream, double *macs) {
  return guarded([&] {
    deconv(h, in_size, out_size, filter, stride, in, out, weight, bias, n_in, n_out, groups, nullptr, nullptr, stream,
           macs);
  });
}
int scn_conv_bn_fwd(scn_metadata *h, int kind, const int64_t *a, const int64_t *b, const int64_t *c,
                    const int64_t *d, const float *in, float *out, const float *weight, const float *bias,
                    int n_in, int n_out, int groups, const scn_bn_params *pre, const scn_bn_params *post,
                    void *stream, double *macs) {
  return guarded([&] {
    BnArgs pre_a{}, post_a{};
    auto conv = [](const scn_bn_params *p, BnArgs &o) -> const BnArgs * {
      if (!p) return nullptr;
      if (!p->running_mean || !p->running_var) throw Error("batch norm parameters need running_mean and running_var");
      o = BnArgs{p->running_mean, p->running_var, p->gamma, p->beta, p->eps, p->leakiness};
      return &o;
    };
    const BnArgs *pa = conv(pre, pre_a), *po = conv(post, post_a);
    if (kind == 0)
      subm_conv(h, a, b, in, out, weight, bias, n_in, n_out, groups, pa, po, stream, macs);
    else if (kind == 1)
      strided_conv(h, a, b, c, d, in, out, weight, bias, n_in, n_out, groups, pa, po, stream, macs);
    else if (kind == 2)
      deconv(h, a, b, c, d, in, out, weight, bias, n_in, n_out, groups, pa, po, stream, macs);
    else
      throw Error("scn_conv_bn_fwd: kind must be 0 (submanifold), 1 (strided) or 2 (transposed)");
  });
}
int scn_nin_fwd(scn_metadata *h, const float *in, float *out, const float *weight, const float *bias,
                int64_t rows, int n_in, int n_out, void *stream, double *macs) {
  return guarded([&] {
    Metadata &m = md(h);
    if (rows < 0 || rows >= ((int64_t)1 << 31)) throw Error("network in network: row count out of range");
    Table *tp;
    {
      BuildScope b(m, stream);
      tp = &identity_table(m, rows, b.s());
    }
    consume(m, st(stream));
    Table &t = *tp;
    conv_forward(m, t, in, rows, out, weight, bias, n_in, n_out, 1, nullptr, nullptr, st(stream));
    // CPU/NetworkInNetwork.cpp:22: nActive * input_nPlanes * output_nPlanes
    note_macs(m, t, (double)n_in * n_out, macs, st(stream));
  });
}
int scn_maxpool_fwd(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *size,
                    const int64_t *stride, const float *in, int in_stride, float *out, int planes,
                    int n_features_to_drop, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    if (planes != in_stride - n_features_to_drop) throw Error("planes must equal in_stride - n_features_to_drop");
    StridedRules &r = strided_table(m, in_size, out_size, size, stride, stream);
    maxpool_forward(r.by_out, in, in_stride, out, planes, n_features_to_drop, st(stream));
  });
}
int scn_avgpool_fwd(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *size,
                    const int64_t *stride, const float *in, int in_stride, float *out, int planes,
                    int n_features_to_drop, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    if (planes != in_stride - n_features_to_drop) throw Error("planes must equal in_stride - n_features_to_drop");
    StridedRules &r = strided_table(m, in_size, out_size, size, stride, stream);
    avgpool_forward(r.by_out, in, in_stride, out, planes, n_features_to_drop, st(stream));
  });
}
int scn_unpool_fwd(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *size,
                   const int64_t *stride, const float *in, int in_stride, float *out, int planes,
                   int n_features_to_drop, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    if (planes != in_stride - n_features_to_drop) throw Error("planes must equal in_stride - n_features_to_drop");
    // CPU/UnPooling.cpp:43-44: the rulebook of (out_size -> in_size), read from the fine side
    StridedRules &r = strided_table_fine(m, out_size, in_size, size, stride, stream);
    unpool_forward(r.by_in, in, in_stride, out, planes, n_features_to_drop, st(stream));
  });
}
int scn_bn_eval_fwd(const float *in, float *out, int64_t rows, int planes, int64_t in_stride,
                    int64_t out_stride, const float *running_mean, const float *running_var,
                    const float *gamma, const float *beta, float eps, float leakiness, void *stream) {
  return guarded([&] {
    bn_eval_forward(in, out, rows, planes, in_stride, out_stride, running_mean, running_var, gamma, beta,
                    eps, leakiness, st(stream));
  });
}
int scn_s2d_fwd(scn_metadata *h, const int64_t *spatial, const float *in, float *out, int planes,
                void *stream) {
  return guarded([&] {
    Level *l = find_level(md(h), spatial);
    if (!l) throw Error("sparse to dense: unknown spatial size");
    consume(md(h), st(stream));
    s2d_forward(*l, in, out, planes, st(stream));
  });
}

scn_params *scn_params_create(void) {
  try {
    return new scn_params();
  } catch (const std::exception &e) {
    g_error = e.what();
    return nullptr;
  }
}
// A parameter set's buffers go back to the cache tagged with the stream they were last used on.
static void tag_params_stream(scn_params *p) {
  if (p && p->p.last_known) pool_set_stream(POOL_COMPUTE, p->p.last);
}
void scn_params_destroy(scn_params *p) {
  tag_params_stream(p);
  delete p;
}
int scn_params_clear(scn_params *p) {
  return guarded([&] {
    if (!p) throw Error("null parameter set");
    tag_params_stream(p);
    p->p.clear();
  });
}
int scn_md_use_params(scn_metadata *h, scn_params *p) {
  return guarded([&] { md(h).frozen = p ? &p->p : nullptr; });
}
int scn_active_pooling_fwd(scn_metadata *h, const int64_t *spatial, const float *in, float *out, int planes,
                           int average, void *stream) {
  return guarded([&] {
    Level *l = find_level(md(h), spatial);
    if (!l) throw Error("active pooling: unknown spatial size");
    consume(md(h), st(stream));
    active_pool_forward(md(h), *l, in, out, planes, average, st(stream));
  });
}
int scn_active_pooling_bwd(scn_metadata *h, const int64_t *spatial, float *d_in, const float *d_out, int planes,
                           int average, void *stream) {
  return guarded([&] {
    Level *l = find_level(md(h), spatial);
    if (!l) throw Error("active pooling: unknown spatial size");
    consume(md(h), st(stream));
    active_pool_backward(md(h), *l, d_in, d_out, planes, average, st(stream));
  });
}

// ---- backward pass -----------------------------------------------------------------------------

int scn_subm_conv_bwd(scn_metadata *h, const int64_t *spatial, const int64_t *filter, const float *in, float *d_in,
                      const float *d_out, const float *weight, float *d_weight, float *d_bias, int n_in,
                      int n_out, int groups, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    Table &t = subm_table(m, spatial, filter, stream);
    subm_conv_backward(m, t, filter, in, d_in, d_out, weight, d_weight, d_bias, n_in, n_out, groups, st(stream));
  });
}
int scn_conv_bwd(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *filter,
                 const int64_t *stride, const float *in, float *d_in, const float *d_out, const float *weight,
                 float *d_weight, float *d_bias, int n_in, int n_out, int groups, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    StridedRules &r = strided_table_fine(m, in_size, out_size, filter, stride, stream);
    strided_conv_backward(m, r.by_out, r.by_in, level_rows(m, in_size), level_rows(m, out_size), in, d_in, d_out,
                          weight, d_weight, d_bias, n_in, n_out, groups, st(stream));
  });
}
int scn_deconv_bwd(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *filter,
                   const int64_t *stride, const float *in, float *d_in, const float *d_out, const float *weight,
                   float *d_weight, float *d_bias, int n_in, int n_out, int groups, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    // CPU/Deconvolution.cpp:56-57: the rulebook of (out_size -> in_size)
    StridedRules &r = strided_table_fine(m, out_size, in_size, filter, stride, stream);
    strided_conv_backward(m, r.by_in, r.by_out, level_rows(m, in_size), level_rows(m, out_size), in, d_in, d_out,
                          weight, d_weight, d_bias, n_in, n_out, groups, st(stream));
  });
}
int scn_nin_bwd(scn_metadata *h, const float *in, float *d_in, const float *d_out, const float *weight,
                float *d_weight, float *d_bias, int64_t rows, int n_in, int n_out, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    if (rows < 0 || rows >= ((int64_t)1 << 31)) throw Error("network in network: row count out of range");
    Table *tp;
    {
      BuildScope b(m, stream);
      tp = &identity_table(m, rows, b.s());
    }
    consume(m, st(stream));
    nin_backward(m, *tp, in, d_in, d_out, weight, d_weight, d_bias, n_in, n_out, st(stream));
  });
}
int scn_bn_train_fwd(scn_metadata *h, const float *in, float *out, int64_t rows, int planes, int64_t in_stride,
                     int64_t out_stride, float *save_mean, float *save_invstd, float *running_mean,
                     float *running_var, const float *gamma, const float *beta, float eps, float momentum,
                     float leakiness, void *stream) {
  return guarded([&] {
    bn_train_forward(&md(h), in, out, rows, planes, in_stride, out_stride, save_mean, save_invstd, running_mean,
                     running_var, gamma, beta, eps, momentum, leakiness, st(stream));
  });
}
int scn_bn_bwd(scn_metadata *h, const float *in, float *d_in, const float *out, const float *d_out, int64_t rows,
               int planes, int64_t in_stride, int64_t out_stride, const float *save_mean, const float *save_invstd,
               const float *gamma, float *d_gamma, float *d_beta, float leakiness, void *stream) {
  return guarded([&] {
    bn_backward(&md(h), in, d_in, out, d_out, rows, planes, in_stride, out_stride, save_mean, save_invstd, gamma,
                d_gamma, d_beta, leakiness, st(stream));
  });
}
int scn_maxpool_bwd(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *size,
                    const int64_t *stride, const float *in, float *d_in, int in_stride, const float *out,
                    const float *d_out, int planes, int n_features_to_drop, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    if (planes != in_stride - n_features_to_drop) throw Error("planes must equal in_stride - n_features_to_drop");
    StridedRules &r = strided_table_fine(m, in_size, out_size, size, stride, stream);
    pool_backward(0, r.by_in, in, d_in, in_stride, out, d_out, planes, n_features_to_drop, st(stream));
  });
}
int scn_avgpool_bwd(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *size,
                    const int64_t *stride, float *d_in, int in_stride, const float *d_out, int planes,
                    int n_features_to_drop, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    if (planes != in_stride - n_features_to_drop) throw Error("planes must equal in_stride - n_features_to_drop");
    StridedRules &r = strided_table_fine(m, in_size, out_size, size, stride, stream);
    pool_backward(1, r.by_in, nullptr, d_in, in_stride, nullptr, d_out, planes, n_features_to_drop, st(stream));
  });
}
int scn_unpool_bwd(scn_metadata *h, const int64_t *in_size, const int64_t *out_size, const int64_t *size,
                   const int64_t *stride, float *d_in, int in_stride, const float *d_out, int planes,
                   int n_features_to_drop, void *stream) {
  return guarded([&] {
    Metadata &m = md(h);
    if (planes != in_stride - n_features_to_drop) throw Error("planes must equal in_stride - n_features_to_drop");
    // CPU/UnPooling.cpp:68-69: the rulebook of (out_size -> in_size); the gradient is gathered from the coarse side
    StridedRules &r = strided_table(m, out_size, in_size, size, stride, stream);
    pool_backward(2, r.by_out, nullptr, d_in, in_stride, nullptr, d_out, planes, n_features_to_drop, st(stream));
  });
}
int scn_input_layer_bwd(scn_metadata *h, float *d_in, const float *d_out, int planes, void *stream) {
  return guarded([&] {
    consume(md(h), st(stream));
    input_backward(md(h).input, d_in, d_out, planes, st(stream));
  });
}
int scn_output_layer_bwd(scn_metadata *h, float *d_in, const float *d_out, int planes, void *stream) {
  return guarded([&] {
    consume(md(h), st(stream));
    output_backward(md(h).input, d_in, d_out, planes, st(stream));
  });
}
int scn_s2d_bwd(scn_metadata *h, const int64_t *spatial, float *d_in, const float *d_out, int planes, void *stream) {
  return guarded([&] {
    Level *l = find_level(md(h), spatial);
    if (!l) throw Error("sparse to dense: unknown spatial size");
    consume(md(h), st(stream));
    s2d_backward(*l, d_in, d_out, planes, st(stream));
  });
}

}  // extern "C"
