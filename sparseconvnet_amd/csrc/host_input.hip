// Coordinates handed over in host memory (the reference's calling convention: InputLayer takes a CPU
// LongTensor, sparseconvnet/ioLayers.py:51-65).  int64 x (dim + 1) per point is 32 bytes, of which a
// grid of up to 32767 cells per dimension uses 8: a few host threads narrow the values to int16
// (int32 when a value does not fit) straight into pinned memory, chunk by chunk, and each chunk is
// copied to the device as soon as it is narrowed, so that the transfer of chunk i overlaps the
// narrowing of chunk i + 1.  For 1.3 M points that is 10 MB over PCIe instead of 42 MB from
// pageable memory.  The device kernels read the narrow values (CoordSrc, metadata.h).
#include "metadata.h"

#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <functional>
#include <mutex>
#include <thread>

namespace scn {
namespace {

// A few worker threads for the process, started on first use and never joined (they sleep on a
// condition variable between jobs).  One job at a time: run(fn) calls fn(worker index) on every
// worker and returns when all have finished.
class Workers {
 public:
  static Workers &get() {
    static Workers *w = new Workers();  // never destroyed: the threads may outlive static destruction
    return *w;
  }
  int count() const { return n_; }
  void run(const std::function<void(int)> &fn) {
    std::lock_guard<std::mutex> one_job(job_mutex_);
    {
      std::lock_guard<std::mutex> lock(mu_);
      fn_ = &fn;
      remaining_ = n_;
      generation_++;
    }
    cv_.notify_all();
    std::unique_lock<std::mutex> lock(mu_);
    done_.wait(lock, [&] { return remaining_ == 0; });
    fn_ = nullptr;
  }

 private:
  Workers() {
    const char *e = getenv("SCN_HOST_THREADS");
    int n = e ? atoi(e) : (int)std::min(8u, std::max(1u, std::thread::hardware_concurrency()));
    n_ = std::max(1, std::min(n, 64));
    for (int i = 0; i < n_; i++) std::thread([this, i] { loop(i); }).detach();
  }
  void loop(int index) {
    uint64_t seen = 0;
    for (;;) {
      const std::function<void(int)> *fn;
      {
        std::unique_lock<std::mutex> lock(mu_);
        cv_.wait(lock, [&] { return generation_ != seen; });
        seen = generation_;
        fn = fn_;
      }
      (*fn)(index);
      {
        std::lock_guard<std::mutex> lock(mu_);
        if (--remaining_ == 0) done_.notify_all();
      }
    }
  }
  int n_ = 1;
  std::mutex job_mutex_, mu_;
  std::condition_variable cv_, done_;
  const std::function<void(int)> *fn_ = nullptr;
  int remaining_ = 0;
  uint64_t generation_ = 0;
};

template <class T> bool narrow_chunk(const int64_t *src, T *dst, int64_t count) {
  int64_t bad = 0;
  for (int64_t i = 0; i < count; i++) {
    const int64_t v = src[i];
    const T t = (T)v;
    dst[i] = t;
    bad |= (int64_t)t ^ v;
  }
  return bad == 0;
}
// int32 with saturation: a value beyond int32 stays outside every grid (the device reports it)
void clamp_chunk(const int64_t *src, int32_t *dst, int64_t count) {
  for (int64_t i = 0; i < count; i++) {
    const int64_t v = src[i];
    dst[i] = (int32_t)std::max<int64_t>(INT32_MIN, std::min<int64_t>(INT32_MAX, v));
  }
}

// Pinned staging blocks come in powers of two so that scenes of different sizes share them.
size_t staging_bytes(size_t bytes) {
  size_t p = (size_t)1 << 20;
  while (p < bytes) p <<= 1;
  return p;
}

}  // namespace

// Narrows host[0 .. values) into m.hostcoords on the device (copies enqueued on s) and returns how
// the kernels are to read it.  The pinned block the copies read from is left in m.staging: whoever
// next synchronises on s (the construction does, to learn what it needs on the host) hands it back
// with release_staging.
CoordSrc stage_host_coords(Metadata &m, const int64_t *host, int64_t values, hipStream_t s, bool allow16) {
  if (values <= 0) return CoordSrc{nullptr, 8};
  Workers &w = Workers::get();
  int device = 0;
  HIP_CHECK(hipGetDevice(&device));
  constexpr int64_t CHUNK = (int64_t)1 << 19;  // values per chunk (1 MB of int16)
  const int64_t chunks = ceil_div(values, CHUNK);
  for (int width = allow16 ? 2 : 4; width <= 4; width += 2) {
    const size_t bytes = (size_t)values * width, block = staging_bytes(bytes);
    m.hostcoords.reserve(bytes);
    release_staging(m);
    m.staging = pinned_acquire(block);
    m.staging_bytes = block;
    unsigned char *pinned = static_cast<unsigned char *>(m.staging);
    std::vector<std::atomic<int>> done(chunks);
    for (auto &d : done) d.store(0, std::memory_order_relaxed);
    std::atomic<int64_t> next{0};
    std::atomic<bool> fits{true}, failed{false};
    const bool copier = w.count() > 1;  // worker 0 enqueues the copies while the others narrow
    w.run([&](int index) {
      if (index == 0 && copier) {  // copies in chunk order, each as soon as its chunk is there
        if (hipSetDevice(device) != hipSuccess) failed.store(true);
        for (int64_t c = 0; c < chunks; c++) {
          while (!done[c].load(std::memory_order_acquire)) std::this_thread::yield();
          if (failed.load() || !fits.load()) continue;
          const int64_t v0 = c * CHUNK, cnt = std::min(CHUNK, values - v0);
          if (hipMemcpyAsync(m.hostcoords.p + v0 * width, pinned + v0 * width, (size_t)cnt * width, hipMemcpyHostToDevice,
                             s) != hipSuccess)
            failed.store(true);
        }
        return;
      }
      for (;;) {
        const int64_t c = next.fetch_add(1);
        if (c >= chunks) break;
        const int64_t v0 = c * CHUNK, cnt = std::min(CHUNK, values - v0);
        if (width == 2) {
          if (!narrow_chunk<int16_t>(host + v0, reinterpret_cast<int16_t *>(pinned) + v0, cnt)) fits.store(false);
        } else {
          clamp_chunk(host + v0, reinterpret_cast<int32_t *>(pinned) + v0, cnt);
        }
        done[c].store(1, std::memory_order_release);
      }
    });
    if (!copier && fits.load() &&
        hipMemcpyAsync(m.hostcoords.p, pinned, bytes, hipMemcpyHostToDevice, s) != hipSuccess)
      failed.store(true);
    if (failed.load()) {
      (void)hipGetLastError();
      (void)hipStreamSynchronize(s);
      release_staging(m);
      throw Error("copying coordinates to the device failed");
    }
    if (fits.load()) return CoordSrc{m.hostcoords.p, width};
    // some value does not fit int16 (a sample index above 32767, or a coordinate the device will
    // refuse): once more with int32, after the copies already enqueued have left the block
    HIP_CHECK(hipStreamSynchronize(s));
  }
  throw Error("internal: coordinates did not narrow");
}

void release_staging(Metadata &m) {
  if (m.staging) pinned_release(m.staging, m.staging_bytes);
  m.staging = nullptr;
  m.staging_bytes = 0;
}

}  // namespace scn
