// Shared by the translation units of the convolution forward (conv.hip: scratch, weight packing,
// dispatch; conv_tiled.hip, conv_rows.hip, conv_resident.hip: one MFMA kernel family each).
#pragma once
#include "metadata.h"

#include <type_traits>

namespace scn {

// Scratch of a convolution (see conv.hip): buffers of the handle, or fixed regions of the static
// array while an allocation-free call runs.
constexpr size_t NOALLOC_QUEUE_BYTES = 4096;              // set counters (8 x 128 bytes used)
constexpr size_t NOALLOC_WPACK_BYTES = (size_t)8 << 20;   // packed weights: 27 taps of 256 x 256 are 7.1 MB
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)16 << 20;
constexpr size_t NOALLOC_PARTIAL_BYTES = NOALLOC_SCRATCH_BYTES - NOALLOC_WPACK_BYTES - NOALLOC_QUEUE_BYTES;
float *scratch_wpack(Metadata &m, size_t floats);
int *scratch_queue(Metadata &m, hipStream_t s);
float *scratch_partial(Metadata &m, int &n_split, int64_t split_stride_floats);

// The weights of the running convolution in the layout `key` names, `floats` long: from the
// caller's frozen set when there is one (packed by `pack(dst)` the first time), else packed into
// the handle's scratch on every call.
template <class F>
static float *packed_weights(Metadata &m, std::vector<int64_t> key, size_t floats, F pack) {
  auto first = [&] {
    if (m.before_pack) m.before_pack();
    m.before_pack = nullptr;
  };
  if (m.frozen && !m.fixed_scratch) {
    if (m.wkey_ptr) {  // a column range: keyed by where it lies in the caller's weights, not by the scratch copy's address
      key[1] += m.wkey_ptr - m.wkey_from;
      key.push_back(m.wkey_c0);
      key.push_back(m.wkey_wc);
    }
    auto it = m.frozen->packed.find(key);
    if (it != m.frozen->packed.end() && it->second.cap >= floats) return it->second.p;
    DevBuf<float> &b = m.frozen->packed[key];
    b.reserve(floats);
    first();
    pack(b.p);
    return b.p;
  }
  float *dst = scratch_wpack(m, floats);
  first();
  pack(dst);
  return dst;
}

typedef float v4f __attribute__((ext_vector_type(4)));
// Four bf16 values in two registers: the A / B operand of v_mfma_f32_16x16x16_bf16, which
// contracts the 16 channels that four fp32 MFMAs (16x16x4) take one after the other.  A lane
// holds the same four consecutive channels in both layouts, so the reduced-precision kernels
// differ from the fp32 ones only in a conversion (round to nearest even) where operands enter
// LDS or the A registers, and in one MFMA instead of four.
typedef short v4s __attribute__((ext_vector_type(4)));
typedef __bf16 v4bf __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
__device__ inline v4s to_bf16x4(v4f v) { return __builtin_bit_cast(v4s, __builtin_convertvector(v, v4bf)); }
// The bf16 kernels take two 16-channel steps per v_mfma_f32_16x16x32_bf16: lane group g
// contributes its four channels of either step (the instruction sums over all 32 (lane group,
// element) pairs, in whatever order A and B agree on).  Operands of a pair of steps are kept
// next to each other (16 bytes per lane) in LDS and in the packed weights, so that they
// arrive in the four consecutive registers the instruction wants.
__device__ inline v8s to_bf16x8(v4f lo, v4f hi) {
  return __builtin_shufflevector(to_bf16x4(lo), to_bf16x4(hi), 0, 1, 2, 3, 4, 5, 6, 7);
}
__device__ inline v4f mfma_bf16(v8s a, v8s b, v4f acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), acc, 0, 0, 0);
}

template <bool PRE> __device__ inline v4f pre_act(v4f v, v4f sc, v4f sh, float leak) {
  if (!PRE) return v;
  v4f y = v * sc + sh;
  y.x *= (y.x > 0.f ? 1.f : leak);
  y.y *= (y.y > 0.f ? 1.f : leak);
  y.z *= (y.z > 0.f ? 1.f : leak);
  y.w *= (y.w > 0.f ? 1.f : leak);
  return y;
}
// Hands the pending jobs to the launch being prepared (and forgets them).
static inline CoefJobs take_jobs(Metadata &m) {
  CoefJobs j = m.jobs;
  m.jobs = CoefJobs();
  return j;
}

// Elements of one packed weight slab (SS steps of 16 channels by NCB column blocks), padded to
// a multiple of 256 lanes' worth so that a workgroup stages it without bounds checks.
constexpr int packed_slab_floats(int SS, int NCB) { return (SS * NCB * 64 + 255) / 256 * 256 * 4; }


// Profiling build (-DSCN_PHASES, see build.py's SCN_EXTRA_FLAGS): thread 0 of every 16th workgroup
// of a tiled kernel stamps the 100 MHz wall clock at up to seven points of its life into its
// translation unit's g_phase_stamps; slot 7 holds the tile's iteration count.  SCN_PHASE_EXPORT(name)
// defines the extern "C" function that copies the stamps to the host.  Compiled out otherwise.
#ifdef SCN_PHASES
static __device__ unsigned long long g_phase_stamps[64 * 8];
#define SCN_PHASE_SLOT() (blockIdx.y == 0 && (blockIdx.x % 16) == 0 && blockIdx.x / 16 < 64 && threadIdx.x == 0)
#define SCN_PHASE(i) do { if (SCN_PHASE_SLOT()) g_phase_stamps[(blockIdx.x / 16) * 8 + (i)] = wall_clock64(); } while (0)
#define SCN_PHASE_VALUE(i, v) do { if (SCN_PHASE_SLOT()) g_phase_stamps[(blockIdx.x / 16) * 8 + (i)] = (unsigned long long)(v); } while (0)
#define SCN_PHASE_EXPORT(name) \
  extern "C" int name(unsigned long long *out) { return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_phase_stamps), sizeof(g_phase_stamps)); }
#else
#define SCN_PHASE(i)
#define SCN_PHASE_VALUE(i, v)
#define SCN_PHASE_EXPORT(name)
#endif

// Notes the kernel a convolution call launches (Metadata::last_kernel).
inline void note_kernel(Metadata &m, const char *family, std::initializer_list<std::pair<const char *, int>> params) {
  std::string t = family;
  for (auto &p : params) t += std::string(" ") + p.first + "=" + std::to_string(p.second);
  if (!m.last_kernel.empty() && m.last_kernel.back() == '+') m.last_kernel += " " + t;  // column ranges, channel parts
  else m.last_kernel = t;
}

struct PreArgs {  // device pointers to the padded coefficient arrays, or nulls
  const float *sc = nullptr, *sh = nullptr;
  float leak = 1.0f;
};

// What a tile's workgroup (NT threads, G granules of 16 positions from position tbase on) sets up
// before its tap loop: the tile's neighbour rows in LDS, jtab[(granule * K + tap) * 16 + row], the
// granules that have each tap, gmask[tap], and the list of the taps any of its rows has (of those
// this workgroup is to take when the taps of a tile are dealt over n_split workgroups: tap k
// belongs to workgroup k % n_split).  Every thread of the workgroup calls it; it ends with a
// barrier and returns the length of the list.
// The table is read tap by tap, 16 * G consecutive entries each, and all of a thread's loads
// (up to eight) are in flight together: a loop of load - store - ballot steps paid one memory
// latency per step, 5 us for 27 taps where the whole convolution of a small level takes 20.
template <int NT, int G>
__device__ inline int tile_setup(const int *__restrict__ nbr, int K, int64_t n, int64_t npad, int64_t tbase, int n_split,
                                 int split, int *jtab, unsigned *gmask, int *taplist, int *ntaps_p) {
  constexpr int PER_TAP = G * 16;          // entries of one tap
  static_assert(NT % PER_TAP == 0 || PER_TAP % NT == 0, "threads and tile rows must divide one another");
  for (int k = threadIdx.x; k < K; k += NT) gmask[k] = 0u;
  __syncthreads();
  const int total = K * PER_TAP;
  constexpr int BATCH = 8;
  for (int e0 = 0; e0 < total; e0 += BATCH * NT) {
    int jv[BATCH];
#pragma unroll
    for (int i = 0; i < BATCH; i++) {
      const int e = e0 + i * NT + (int)threadIdx.x;
      const int k = e / PER_TAP, p = e % PER_TAP;
      jv[i] = -1;
      if (e < total && tbase + p < n) jv[i] = nbr[(int64_t)k * npad + tbase + p];
    }
#pragma unroll
    for (int i = 0; i < BATCH; i++) {
      const int e = e0 + i * NT + (int)threadIdx.x;
      const int k = e / PER_TAP, p = e % PER_TAP;
      if (e < total) jtab[((p >> 4) * K + k) * 16 + (p & 15)] = jv[i];
      // sixteen consecutive lanes hold one granule's rows of one tap
      const unsigned long long bal = __ballot(jv[i] >= 0);
      const int lane = threadIdx.x & 63;
      if ((lane & 15) == 0 && e < total && ((bal >> lane) & 0xFFFFull)) atomicOr(&gmask[k], 1u << (p >> 4));
    }
  }
  __syncthreads();
  if (threadIdx.x < 64) {  // the first wavefront lists the taps, 64 at a time, in ascending order
    int count = 0;
    for (int k0 = 0; k0 < K; k0 += 64) {
      const int k = k0 + (int)threadIdx.x;
      const bool mine = k < K && gmask[k] != 0u && (n_split == 1 || k % n_split == split);
      const unsigned long long bal = __ballot(mine);
      if (mine) taplist[count + __popcll(bal & ((1ull << threadIdx.x) - 1ull))] = k;
      count += __popcll(bal);
    }
    if (threadIdx.x == 0) *ntaps_p = count;
  }
  __syncthreads();
  return *ntaps_p;
}

// Launchers of the kernels conv.hip defines for the other translation units.
// k_pack_weights / k_pack_weights_part / k_pack_weights_c4: weights into MFMA B-operand order.
void launch_pack_weights(const float *w, float *wp, int K, int n_in, int n_out, int n_slab, int SS, int NCB,
                         int slab_stride, CoefJobs jobs, bool as_bf16, hipStream_t s);
void launch_pack_weights_part(const float *w, float *wp, int K, int w_rows, int n_in_part, int n_out, int SS, int NCB,
                              int *queue, CoefJobs jobs, bool as_bf16, hipStream_t s);
void launch_pack_weights_c4(const float *w, float *wp, int K, int n_in, int n_out, int NCB, int *queue, CoefJobs jobs,
                            hipStream_t s);
// out[rowmap[pos]][col] = epilogue(bias[col] + sum over splits of partial[split][pos][col])
void launch_conv_reduce(const float *partial, int n_split, int64_t split_stride, int ld, const int *rowmap, int64_t n,
                        Epi epi, float *out, int n_out, hipStream_t s);

// The three MFMA kernel families; each returns false when it has no instantiation for the shape.
bool conv_tiled_dispatch(bool vec4, bool pre_fused, Metadata &m, const Table &t, const float *in, float *out,
                         const float *w, Epi epi, int n_in, int n_out, PreArgs pre, hipStream_t s);
bool conv_rows_dispatch(bool vec4, bool pre_fused, Metadata &m, const Table &t, const float *in, float *out,
                        const float *w, Epi epi, int n_in, int n_out, PreArgs pre, hipStream_t s);
// conv_few.hip: transposed convolutions of filter = stride = 2 rulebooks whose weights fit LDS.
bool try_few(Metadata &m, const Table &t, const float *in, float *out, const float *w, Epi epi, int n_in, int n_out,
             hipStream_t s);
bool resident_fits(const Metadata &m, const Table &t, int n_in, int n_out, bool with_bn);
bool try_resident(Metadata &m, const Table &t, const float *in, float *out, const float *w, Epi epi, int n_in,
                  int n_out, hipStream_t s);

}  // namespace scn
