// Convolution forward, output-stationary: every output row accumulates, over the filter
// taps, the row its neighbour table names times that tap's weight slice, and is written
// exactly once (no atomics, no read-modify-write of the output, deterministic).
// One kernel family serves SubmanifoldConvolution, Convolution and Deconvolution
// (CPU/Convolution.cpp:45-79,117-150, CPU/Deconvolution.cpp:7-41); they differ only in
// the table they pass.
//
// Three MFMA kernels (groups == 1, fp32 v_mfma_f32_16x16x4_f32, accumulators in registers
// for the whole filter, taps skipped per 16-row granule), chosen by the output width:
//   k_conv_resident  nOut <= 32   all taps' weights resident in LDS, wavefronts run alone
//   k_conv_rows      nOut <= 128  wavefronts own rows, the weight slab goes through LDS
//   k_conv_mfma      wider        wavefronts own columns, rows and weights go through LDS
// and k_conv_generic for everything else (groups > 1).  Positions arrive in Z-order and
// pattern-sorted, so a granule's rows mostly share one neighbour pattern and the skipped
// (granule, tap) pairs carry almost all of the sparsity.  Template flag BUF: the gathers are
// buffer loads, for which an absent row is an offset past the end that reads as zeros;
// without it absent rows read row 0 and are zeroed by a select.  PRE / Epi: the batch norm +
// leaky ReLU of the layer in front / behind, applied to the gathered / stored values.
#include "metadata.h"

#include <map>
#include <mutex>
#include <type_traits>

namespace scn {

// ---- scratch of a convolution -------------------------------------------------------------------
// The kernels below need device memory beyond their inputs and outputs: the weights in MFMA
// operand order, the set counters of the resident-weights kernel, and partial tiles when a small
// level's taps are split over workgroups.  Normally these are buffers of the handle, grown on
// demand from the block cache.  The allocation-free entry point (scn_subm_conv_fwd_noalloc) may
// not allocate: it takes them from this array instead, one copy per GPU, held until the process
// ends and shared by every such call on that GPU (overlapping calls on one GPU race).
constexpr size_t NOALLOC_QUEUE_BYTES = 4096;              // set counters (8 x 128 bytes used)
constexpr size_t NOALLOC_WPACK_BYTES = (size_t)8 << 20;   // packed weights: 27 taps of 256 x 256 are 7.1 MB
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)16 << 20;
constexpr size_t NOALLOC_PARTIAL_BYTES = NOALLOC_SCRATCH_BYTES - NOALLOC_WPACK_BYTES - NOALLOC_QUEUE_BYTES;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

// The array's address on the current device.  In host code the array's name is only a handle
// for the runtime; the address kernels can use comes from hipGetSymbolAddress, once per device.
unsigned char *noalloc_scratch() {
  static std::mutex mu;
  static std::map<int, unsigned char *> ptrs;
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  auto it = ptrs.find(dev);
  if (it != ptrs.end()) return it->second;
  void *p = nullptr;
  HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
  if (!p) throw Error("the scratch array has no address on this device");
  return ptrs[dev] = static_cast<unsigned char *>(p);
}

static float *scratch_wpack(Metadata &m, size_t floats) {
  if (m.fixed_scratch) {
    if (floats * sizeof(float) > NOALLOC_WPACK_BYTES)
      throw Error("allocation-free convolution: the packed weights (taps x input planes x output planes x 4 bytes, "
                  "padded to 16 x 16 blocks) exceed the 8 MiB the static scratch holds");
    return reinterpret_cast<float *>(m.fixed_scratch + NOALLOC_QUEUE_BYTES);
  }
  m.wpack.reserve(floats);
  return m.wpack.p;
}
// Nine counters 128 bytes apart: one per XCD for the sets handed out, one for the workgroups that
// have finished.  They are zero between launches: static device memory starts as zeros, the
// handle's buffer is cleared when it is allocated, and the last workgroup of every launch clears
// them again.
static int *scratch_queue(Metadata &m, hipStream_t s) {
  if (m.fixed_scratch) return reinterpret_cast<int *>(m.fixed_scratch);
  if (!m.queue_zeroed) {
    m.queue.reserve(9 * 32);
    fill32(m.queue.p, 0, 9 * 32, s);
    m.queue_zeroed = true;
  }
  return m.queue.p;
}
// The weights of the running convolution in the layout `key` names, `floats` long: from the
// caller's frozen set when there is one (packed by `pack(dst)` the first time), else packed into
// the handle's scratch on every call.
template <class F>
static float *packed_weights(Metadata &m, std::vector<int64_t> key, size_t floats, F pack) {
  if (m.frozen && !m.fixed_scratch) {
    auto it = m.frozen->packed.find(key);
    if (it != m.frozen->packed.end() && it->second.cap >= floats) return it->second.p;
    DevBuf<float> &b = m.frozen->packed[key];
    b.reserve(floats);
    pack(b.p);
    return b.p;
  }
  float *dst = scratch_wpack(m, floats);
  pack(dst);
  return dst;
}
// Partial tiles for n_split workgroups per tile; with the static scratch n_split shrinks until
// they fit (1: no partial tiles at all).
static float *scratch_partial(Metadata &m, int &n_split, int64_t split_stride_floats) {
  if (m.fixed_scratch) {
    const int64_t fit = (int64_t)(NOALLOC_PARTIAL_BYTES / sizeof(float)) / std::max<int64_t>(split_stride_floats, 1);
    n_split = (int)std::max<int64_t>(1, std::min<int64_t>(n_split, fit));
    return n_split > 1 ? reinterpret_cast<float *>(m.fixed_scratch + NOALLOC_QUEUE_BYTES + NOALLOC_WPACK_BYTES) : nullptr;
  }
  if (n_split <= 1) return nullptr;
  m.partial.reserve((size_t)n_split * split_stride_floats);
  return m.partial.p;
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
__global__ void k_coefs(CoefJobs jobs) { coef_jobs(jobs); }
// Hands the pending jobs to the launch being prepared (and forgets them).
static CoefJobs take_jobs(Metadata &m) {
  CoefJobs j = m.jobs;
  m.jobs = CoefJobs();
  return j;
}

// ---- generic kernel: any channel counts, any groups -------------------------------------
__global__ void k_conv_generic(const int *nbr, const int *rowmap, int K, int64_t n, int64_t npad,
                               const float *in, float *out, const float *w, Epi epi, int n_in,
                               int n_out, int groups) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = n * n_out;
  if (i >= total) return;
  int64_t t = i / n_out;
  int oc = (int)(i - t * n_out);
  int ip = n_in / groups, op = n_out / groups;
  int g = oc / op, ocg = oc - g * op;
  float acc = epi.bias ? epi.bias[oc] : 0.0f;
  for (int k = 0; k < K; k++) {
    int j = nbr[(int64_t)k * npad + t];
    if (j < 0) continue;
    const float *x = in + (int64_t)j * n_in + g * ip;
    const float *wk = w + (((int64_t)k * groups + g) * ip) * op + ocg;
    float a = 0.0f;
    for (int c = 0; c < ip; c++) a += x[c] * wk[(int64_t)c * op];
    acc += a;
  }
  if (epi.sc) acc = epi_act(acc, epi.sc[oc], epi.sh[oc], epi.leak);
  int64_t row = rowmap ? rowmap[t] : t;
  out[row * n_out + oc] = acc;
}

// Elements of one packed weight slab (SS steps of 16 channels by NCB column blocks), padded to
// a multiple of 256 lanes' worth so that a workgroup stages it without bounds checks.
constexpr int packed_slab_floats(int SS, int NCB) { return (SS * NCB * 64 + 255) / 256 * 256 * 4; }

// ---- weight packing ---------------------------------------------------------------------
// wp[k][slab][e], e < SLAB_STRIDE (floats), with for e = ((s*NCB + cb)*64 + lane)*4 + jj
//   wp = W[k][channel (slab*SS+s)*16 + 4*(lane/16) + jj][16*cb + lane%16]
// (zero outside [nIn) x [nOut) and in the padding up to SLAB_STRIDE): the order in which
// lane `lane` of a wavefront consumes B operands, so that staging a slab into LDS is a
// straight copy and each lane reads the four operands of one 16-channel step with a single
// 16-byte LDS load.
// as_bf16 (SS even): 2-byte elements rounded to nearest even, the two steps of a pair next to
// each other: e = (((sp*NCB + cb)*64 + lane)*2 + s%2)*4 + jj with sp = s/2.
__global__ void k_pack_weights(const float *w, float *wp, int K, int n_in, int n_out, int n_slab, int SS,
                               int NCB, int slab_stride, CoefJobs jobs, bool as_bf16 = false) {
  coef_jobs(jobs);
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)K * n_slab * slab_stride;
  if (i >= total) return;
  int e = (int)(i % slab_stride);
  int64_t r = i / slab_stride;
  int sl = (int)(r % n_slab);
  int k = (int)(r / n_slab);
  float v = 0.0f;
  if (e < SS * NCB * 256) {
    int jj = e & 3;
    int lane = (e >> 2) & 63;
    int q = e >> 8;
    int cb = q % NCB;
    int s = q / NCB;
    if (as_bf16) {
      lane = (e >> 3) & 63;
      q = e >> 9;
      cb = q % NCB;
      s = 2 * (q / NCB) + ((e >> 2) & 1);
    }
    int ch = (sl * SS + s) * 16 + 4 * (lane >> 4) + jj;
    int col = 16 * cb + (lane & 15);
    if (ch < n_in && col < n_out) v = w[((int64_t)k * n_in + ch) * n_out + col];
  }
  if (as_bf16)
    reinterpret_cast<__bf16 *>(wp)[i] = (__bf16)v;
  else
    wp[i] = v;
}

// Packs rows [0, n_in_part) of every tap's weight slice, where the slice of tap k starts at
// w + k * w_rows * n_out (w already points at the first row of the range), as one slab per tap
// in the layout of k_pack_weights.
// Also clears the eight set counters (one per XCD, 128 bytes apart) of the launch it precedes.
__global__ void k_pack_weights_part(const float *w, float *wp, int K, int w_rows, int n_in_part, int n_out,
                                    int SS, int NCB, int *queue, CoefJobs jobs, bool as_bf16 = false) {
  coef_jobs(jobs);
  if (blockIdx.x == 0 && threadIdx.x < 8) queue[threadIdx.x * 32] = 0;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)K * SS * NCB * 256;
  if (i >= total) return;
  int e = (int)(i % (SS * NCB * 256));
  int k = (int)(i / (SS * NCB * 256));
  int jj = e & 3;
  int lane = (e >> 2) & 63;
  int q = e >> 8;
  int cb = q % NCB;
  int s = q / NCB;
  if (as_bf16) {  // pairs of steps next to each other, 2-byte elements (see k_pack_weights)
    lane = (e >> 3) & 63;
    q = e >> 9;
    cb = q % NCB;
    s = 2 * (q / NCB) + ((e >> 2) & 1);
  }
  int ch = s * 16 + 4 * (lane >> 4) + jj;
  int col = 16 * cb + (lane & 15);
  const float v = (ch < n_in_part && col < n_out) ? w[((int64_t)k * w_rows + ch) * n_out + col] : 0.0f;
  if (as_bf16)
    reinterpret_cast<__bf16 *>(wp)[i] = (__bf16)v;
  else
    wp[i] = v;
}

// ---- MFMA kernel ------------------------------------------------------------------------
// A workgroup of 4 wavefronts owns a tile of G = GW*WR granules (16 rows each).  The
// wavefronts form a WR x WC grid: wavefront (wr, wc) keeps, in registers, the accumulators
// of granules [wr*GW, (wr+1)*GW) x column blocks [wc*NCBW, (wc+1)*NCBW) (16 columns each).
// With WC = 4 every wavefront works on every granule, so the MFMA work of a tap is split
// evenly whatever the neighbour pattern of the rows.
//
// Per (tap, slab of SS*16 input channels) iteration, for the granules that have the tap:
//   gathered input rows  HBM/L2 -> registers -> LDS, in A-operand order
//   the weight slab      HBM/L2 -> registers -> LDS, in B-operand order (see k_pack_weights)
//   MFMAs out of LDS into the accumulators
// as a software pipeline with one barrier per iteration: iteration it+1's loads are in
// flight while iteration it computes; both LDS areas are double-buffered.  Every global
// load of the pipeline is unconditional (granules without the tap and absent rows read
// row 0 and are zeroed by a select), so the count of loads in flight is a compile-time
// constant and the compiler can wait for exactly the loads it needs.
template <int NCBW, int WC, int GW, int SS, bool VEC4, bool PRE, bool BUF, bool BF16>
__global__ __launch_bounds__(256, 2) void k_conv_mfma(
    const int *__restrict__ nbr, const int *__restrict__ rowmap, int K, int64_t n, int64_t npad,
    const float *__restrict__ in, float *__restrict__ out, const float *__restrict__ wp,
    Epi epi, int n_in, int n_out, int n_slab, int tiles_per_xcd, int n_tiles,
    int n_split, float *__restrict__ partial, const float *__restrict__ pre_sc,
    const float *__restrict__ pre_sh, float pre_leak, unsigned in_bytes) {
  static_assert(!BUF || VEC4, "buffer gathers need float4 rows");
  static_assert(!BF16 || (BUF && SS % 2 == 0), "the bf16 variant: buffer gathers, steps in pairs");
  constexpr int WR = 4 / WC;
  constexpr int NCB = NCBW * WC;
  constexpr int G = GW * WR;
  constexpr int TM = G * 16;
  // An operand is what one lane feeds one MFMA with: 16 bytes, either four fp32 channels of
  // one 16-channel step or four bf16 channels of each step of a pair.
  constexpr int WS = BF16 ? SS / 2 : SS;      // operands per slab, column block and lane
  constexpr int SLAB_STRIDE_F4 = packed_slab_floats(SS, NCB) / (BF16 ? 8 : 4);  // slab in global memory
  constexpr int NFRAG = G * SS;               // A fragments (granule, step) per iteration
  constexpr int FPW = NFRAG / 4;              // fragments gathered per wavefront
  constexpr int A_F4 = G * WS * 64;           // A operands per iteration
  static_assert(NFRAG % 4 == 0, "fragments must divide over 4 wavefronts");
  extern __shared__ __attribute__((aligned(16))) float lds[];
  v4f *abuf = reinterpret_cast<v4f *>(lds);   // [2][A_F4]
  int *jtab = reinterpret_cast<int *>(abuf + 2 * A_F4);  // [G][K][16]
  unsigned *gmask = reinterpret_cast<unsigned *>(jtab + G * K * 16);  // [K] granules having tap k
  int *taplist = reinterpret_cast<int *>(gmask + K);           // [K]
  int *ntaps_p = taplist + K;                                  // [1]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int wr = wave / WC, wc = wave % WC;

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of
  // tiles so that neighbouring tiles (which gather the same rows) share one L2.
  const int tile = (blockIdx.x & 7) * tiles_per_xcd + (blockIdx.x >> 3);
  if (tile >= n_tiles) return;  // whole workgroup leaves: no barrier is skipped
  const int64_t tbase = (int64_t)tile * TM;

  for (int k = threadIdx.x; k < K; k += 256) gmask[k] = 0u;
  __syncthreads();
  // Neighbour rows of the tile -> LDS, four taps per pass (one per 16-lane group).
  for (int gr = wave; gr < G; gr += 4) {
    const int64_t t = tbase + gr * 16 + r16;
    for (int kb = 0; kb < K; kb += 4) {
      const int k = kb + g;
      int j = -1;
      if (k < K && t < n) j = nbr[(int64_t)k * npad + t];
      if (k < K) jtab[(gr * K + k) * 16 + r16] = j;
      const unsigned long long bal = __ballot(j >= 0);
      if (lane == 0) {
#pragma unroll
        for (int gg = 0; gg < 4; gg++)
          if ((bal >> (16 * gg)) & 0xFFFFull) atomicOr(&gmask[kb + gg], 1u << gr);
      }
    }
  }
  __syncthreads();
  // With n_split > 1 the taps of a tile are dealt over n_split workgroups (blockIdx.y), each
  // of which writes a partial tile that k_conv_reduce sums: small levels have too few tiles
  // to fill the GPU and too long a serial tap loop otherwise.
  if (threadIdx.x == 0) {
    int c = 0;
    for (int k = 0; k < K; k++)
      if (gmask[k] && (n_split == 1 || k % n_split == (int)blockIdx.y)) taplist[c++] = k;
    *ntaps_p = c;
  }
  __syncthreads();
  const int total = *ntaps_p * n_slab;

  v4f acc[GW][NCBW];
#pragma unroll
  for (int q = 0; q < GW; q++)
#pragma unroll
    for (int c = 0; c < NCBW; c++) acc[q][c] = (v4f){0.f, 0.f, 0.f, 0.f};

  // Loads in flight, one iteration ahead.  The weights never pass through LDS: a wavefront's
  // column blocks are its own (wavefronts that share a column range, WR = 2, each fetch their
  // copy from L2), and the packed layout is the lane order of the B operand, so a lane's 16
  // bytes per (step, column block) are one coalesced load.  They alternate between two register
  // sets (iteration parity; the loop is unrolled twice so that the set is a constant), because
  // the set of iteration it+1 is being filled while the MFMAs of iteration it read theirs.
  // The gathered rows go through double-buffered LDS, since every wavefront needs all of them.
  v4f breg[2][WS][NCBW];
  v4f areg[FPW];
  v4f psc[FPW], psh[FPW];           // pre-activation coefficients of the fragments' channels
  unsigned gm_nxt = 0, gm_cur = 0;  // granule mask of the tap (uniform)
  unsigned aok_nxt = 0;             // bit i: this lane's row of fragment i exists
  int sl_nxt = 0;

  // BUF: gathers through buffer loads; an absent row becomes an offset of 2 GiB, which is past
  // the end and reads as zeros (see k_conv_rows).
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(in), 0, BUF ? (int)in_bytes : 0, 0x00020000);
  const unsigned row_bytes = (unsigned)n_in * 4u, lane_off = 16u * (unsigned)g;
  const int ntaps = *ntaps_p;
  // Issue the loads of iteration `it`: this wavefront's weights into register set P (= it % 2)
  // and its share of the A fragments (granule, step) into areg.
  auto issue = [&](int it, auto par_c) {
    constexpr int P = decltype(par_c)::value;
    // Slab outer, tap inner: while a slab is being worked on, the tile and its neighbours in
    // the XCD's range gather the same 64-byte columns of a few hundred rows over and over (a
    // row feeds ~10 taps), a working set that stays in L2; with the tap outermost every
    // gather of a 1 KiB row came from HBM (12 GB per launch at 256 planes).
    const int sl = it / ntaps, ti = it - sl * ntaps;
    // LDS values every lane reads alike: tell the compiler, so that what follows from them
    // (weight address, branches on the granule mask) is scalar work
    const int k = __builtin_amdgcn_readfirstlane(taplist[ti]);
    const unsigned gm = __builtin_amdgcn_readfirstlane(gmask[k]);
    gm_nxt = gm;
    sl_nxt = sl;
    aok_nxt = 0;
    const v4f *wsrc = reinterpret_cast<const v4f *>(wp) + ((int64_t)k * n_slab + sl) * SLAB_STRIDE_F4;
#pragma unroll
    for (int s = 0; s < WS; s++)
#pragma unroll
      for (int c = 0; c < NCBW; c++) breg[P][s][c] = wsrc[(s * NCB + wc * NCBW + c) * 64 + lane];
#pragma unroll
    for (int i = 0; i < FPW; i++) {
      const int f = wave + 4 * i;  // fragment f = (granule f / SS, step f % SS)
      const int gr = f / SS, s = f % SS;
      const int j = jtab[(gr * K + k) * 16 + r16];
      if constexpr (BUF) {
        const unsigned voff = j >= 0 ? __umul24((unsigned)j, row_bytes) + lane_off : 0x80000000u;
        areg[i] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, (sl * SS + s) * 64, 0));
        if (PRE) {  // zero must stay zero through the pre-activation
          if (j >= 0) aok_nxt |= 1u << i;
          psc[i] = *reinterpret_cast<const v4f *>(pre_sc + (sl * SS + s) * 16 + 4 * g);
          psh[i] = *reinterpret_cast<const v4f *>(pre_sh + (sl * SS + s) * 16 + 4 * g);
        }
        continue;
      }
      if (j >= 0) aok_nxt |= 1u << i;
      const float *src = in + (int64_t)(j < 0 ? 0 : j) * n_in;
      const int c0 = (sl * SS + s) * 16 + 4 * g;
      if (PRE) {
        psc[i] = *reinterpret_cast<const v4f *>(pre_sc + c0);
        psh[i] = *reinterpret_cast<const v4f *>(pre_sh + c0);
      }
      v4f v;
      if (VEC4) {
        const int cc = c0 < n_in ? c0 : n_in - 4;
        v = *reinterpret_cast<const v4f *>(src + cc);
      } else {
        v.x = src[min(c0 + 0, n_in - 1)];
        v.y = src[min(c0 + 1, n_in - 1)];
        v.z = src[min(c0 + 2, n_in - 1)];
        v.w = src[min(c0 + 3, n_in - 1)];
      }
      areg[i] = v;
    }
  };

  // One iteration; P = it % 2 selects the LDS buffer of the rows and the weights' register set.
  auto iterate = [&](int it, auto par_c) {
    constexpr int P = decltype(par_c)::value;
    v4f *ab = abuf + P * A_F4;
    // Absent rows and channels past nIn become zeros on their way into LDS.
#pragma unroll
    for (int i = 0; i < FPW; i++) {
      const int f = wave + 4 * i;
      const int c0 = (sl_nxt * SS + f % SS) * 16 + 4 * g;
      const bool ok = (aok_nxt >> i) & 1u;
      v4f v = pre_act<PRE>(areg[i], psc[i], psh[i], pre_leak);
      if (BUF) {
        if (PRE && !ok) v = (v4f){0.f, 0.f, 0.f, 0.f};
      } else if (VEC4) {
        if (!(ok && c0 < n_in)) v = (v4f){0.f, 0.f, 0.f, 0.f};
      } else {
        if (!(ok && c0 + 0 < n_in)) v.x = 0.f;
        if (!(ok && c0 + 1 < n_in)) v.y = 0.f;
        if (!(ok && c0 + 2 < n_in)) v.z = 0.f;
        if (!(ok && c0 + 3 < n_in)) v.w = 0.f;
      }
      if constexpr (BF16)  // the half of the pair's operand that belongs to step f % SS
        reinterpret_cast<v4s *>(ab)[(((f / SS) * WS + (f % SS) / 2) * 64 + lane) * 2 + (f & 1)] = to_bf16x4(v);
      else
        ab[f * 64 + lane] = v;
    }
    gm_cur = gm_nxt;
    // After this barrier the rows of `it` are visible, and every wavefront has finished the
    // MFMAs of it-1, so the other buffer may be overwritten at the top of it+1.
    __syncthreads();
    if (it + 1 < total) issue(it + 1, std::integral_constant<int, 1 - P>{});

    // fp32: all A fragments of this wavefront's granules are fetched before the first MFMA, so
    // that no MFMA waits on LDS.  bf16: a granule's fragment is fetched when its turn comes.
    v4f afrag[BF16 ? 1 : GW][WS];
    if constexpr (!BF16) {
#pragma unroll
      for (int q = 0; q < GW; q++)
#pragma unroll
        for (int s = 0; s < WS; s++) afrag[q][s] = ab[((wr * GW + q) * WS + s) * 64 + lane];
    }
#pragma unroll
    for (int q = 0; q < GW; q++) {
      const int gr = wr * GW + q;
      if (!((gm_cur >> gr) & 1u)) continue;  // uniform over the workgroup
#pragma unroll
      for (int s = 0; s < WS; s++) {
        if constexpr (BF16) {
          const v4f af = ab[((wr * GW + q) * WS + s) * 64 + lane];
#pragma unroll
          for (int c = 0; c < NCBW; c++)
            acc[q][c] = mfma_bf16(__builtin_bit_cast(v8s, af), __builtin_bit_cast(v8s, breg[P][s][c]), acc[q][c]);
        } else {
          const v4f av = afrag[q][s];
#pragma unroll
          for (int c = 0; c < NCBW; c++) acc[q][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, breg[P][s][c].x, acc[q][c], 0, 0, 0);
#pragma unroll
          for (int c = 0; c < NCBW; c++) acc[q][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, breg[P][s][c].y, acc[q][c], 0, 0, 0);
#pragma unroll
          for (int c = 0; c < NCBW; c++) acc[q][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, breg[P][s][c].z, acc[q][c], 0, 0, 0);
#pragma unroll
          for (int c = 0; c < NCBW; c++) acc[q][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, breg[P][s][c].w, acc[q][c], 0, 0, 0);
        }
      }
    }
  };

  if (total > 0) issue(0, std::integral_constant<int, 0>{});
  for (int it = 0; it < total; it += 2) {
    iterate(it, std::integral_constant<int, 0>{});
    if (it + 1 < total) iterate(it + 1, std::integral_constant<int, 1>{});
  }

  // acc[q][c][r] = result for position tbase + 16*(wr*GW+q) + 4*g + r, column 16*(wc*NCBW+c) + r16
  if (partial != nullptr) {  // [n_split][n_tiles * TM][NCB * 16]
    float *pt = partial + ((int64_t)blockIdx.y * n_tiles * TM + tbase) * (NCB * 16);
#pragma unroll
    for (int q = 0; q < GW; q++)
#pragma unroll
      for (int r = 0; r < 4; r++)
#pragma unroll
        for (int c = 0; c < NCBW; c++)
          pt[(int64_t)((wr * GW + q) * 16 + 4 * g + r) * (NCB * 16) + 16 * (wc * NCBW + c) + r16] = acc[q][c][r];
    return;
  }
  float bv[NCBW], es[NCBW], eh[NCBW];
  const bool post = epi.sc != nullptr;
#pragma unroll
  for (int c = 0; c < NCBW; c++) {
    const int col = 16 * (wc * NCBW + c) + r16;
    bv[c] = (epi.bias != nullptr && col < n_out) ? epi.bias[col] : 0.0f;
    es[c] = (post && col < n_out) ? epi.sc[col] : 1.0f;
    eh[c] = (post && col < n_out) ? epi.sh[col] : 0.0f;
  }
#pragma unroll
  for (int q = 0; q < GW; q++) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int64_t pos = tbase + (wr * GW + q) * 16 + 4 * g + r;
      if (pos >= n) continue;
      const int64_t row = rowmap ? rowmap[pos] : pos;
      float *o = out + row * (epi.out_stride ? epi.out_stride : n_out);
#pragma unroll
      for (int c = 0; c < NCBW; c++) {
        const int col = 16 * (wc * NCBW + c) + r16;
        float v = acc[q][c][r] + bv[c];
        if (post) v = epi_act(v, es[c], eh[c], epi.leak);
        if (col < n_out) o[col] = v;
      }
    }
  }
}

// out[rowmap[pos]][col] = epilogue(bias[col] + sum over splits of partial[split][pos][col])
__global__ void k_conv_reduce(const float *partial, int n_split, int64_t split_stride, int ld, const int *rowmap,
                              int64_t n, Epi epi, float *out, int n_out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * n_out) return;
  int64_t pos = i / n_out;
  int col = (int)(i - pos * n_out);
  float acc = epi.bias ? epi.bias[col] : 0.0f;
  for (int sp = 0; sp < n_split; sp++) acc += partial[sp * split_stride + pos * ld + col];
  if (epi.sc) acc = epi_act(acc, epi.sc[col], epi.sh[col], epi.leak);
  int64_t row = rowmap ? rowmap[pos] : pos;
  out[row * (epi.out_stride ? epi.out_stride : n_out) + col] = acc;
}

struct PreArgs {  // device pointers to the padded coefficient arrays, or nulls
  const float *sc = nullptr, *sh = nullptr;
  float leak = 1.0f;
};

template <int NCBW, int WC, int GW, int SS, bool VEC4, bool PRE, bool BUF = false, bool BF16 = false>
static bool launch_mfma(Metadata &m, const Table &t, const float *in, float *out, const float *w,
                        Epi epi, int n_in, int n_out, PreArgs pre, hipStream_t s) {
  if constexpr (VEC4 && !BUF) {
    if (n_in % (16 * SS) == 0 && m.cur_in_rows > 0 && m.cur_in_rows < (1 << 24) &&
        m.cur_in_rows * n_in * 4 < ((int64_t)1 << 31) && n_in * 4 < (1 << 24)) {
      if (m.bf16 && n_in % 32 == 0)  // half-size operands leave room for two steps per slab
        return launch_mfma<NCBW, WC, GW, 2, VEC4, PRE, true, true>(m, t, in, out, w, epi, n_in, n_out, pre, s);
      return launch_mfma<NCBW, WC, GW, SS, VEC4, PRE, true>(m, t, in, out, w, epi, n_in, n_out, pre, s);
    }
  }
  constexpr int WR = 4 / WC, NCB = NCBW * WC, G = GW * WR;
  constexpr int WS = BF16 ? SS / 2 : SS;
  constexpr int SLAB_STRIDE = packed_slab_floats(SS, NCB);  // elements of a packed slab
  const size_t lds_bytes = (size_t)2 * G * WS * 64 * 16 + ((size_t)G * t.K * 16 + 2 * t.K + 4) * sizeof(int);
  if (lds_bytes > 160 * 1024) return false;
  const int cin16 = (int)ceil_div(n_in, 16);
  const int n_slab = (int)ceil_div(cin16, SS);
  const int64_t packed = (int64_t)t.K * n_slab * SLAB_STRIDE;
  float *wpack = packed_weights(m, {0, (int64_t)(uintptr_t)w, t.K, n_in, n_out, SS, NCB, BF16}, packed, [&](float *dst) {
    k_pack_weights<<<dim3((unsigned)ceil_div(packed, 256)), 256, 0, s>>>(w, dst, t.K, n_in, n_out, n_slab, SS, NCB,
                                                                        SLAB_STRIDE, take_jobs(m), BF16);
    LAUNCH_CHECK();
  });
  auto kern = k_conv_mfma<NCBW, WC, GW, SS, VEC4, PRE, BUF, BF16>;
  static bool attr_set = false;
  if (!attr_set) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  160 * 1024));
    attr_set = true;
  }
  const int n_tiles = (int)ceil_div(t.n, G * 16);
  const int tiles_per_xcd = (int)ceil_div(n_tiles, 8);
  // Few tiles: deal the taps of every tile over several workgroups (about two per CU in all).
  int n_split = 1;
  if (n_tiles < 256) n_split = (int)std::min<int64_t>(t.K, ceil_div(512, n_tiles));
  const int64_t split_stride = (int64_t)n_tiles * G * 16 * NCB * 16;
  float *partial = scratch_partial(m, n_split, split_stride);
  kern<<<dim3((unsigned)(tiles_per_xcd * 8), n_split), 256, lds_bytes, s>>>(
      t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, in, out, wpack, epi, n_in, n_out, n_slab, tiles_per_xcd,
      n_tiles, n_split, partial, pre.sc, pre.sh, pre.leak, (unsigned)(m.cur_in_rows * n_in * 4));
  LAUNCH_CHECK();
  if (n_split > 1) {
    k_conv_reduce<<<dim3((unsigned)ceil_div(t.n * n_out, 256)), 256, 0, s>>>(partial, n_split, split_stride, NCB * 16,
                                                                          t.rowmap_ptr(), t.n, epi, out, n_out);
    LAUNCH_CHECK();
  }
  return true;
}

// Picks the instantiation from the number of 16-column blocks of the output.  Tiles are 8
// granules (128 rows); registers and LDS are sized so that two workgroups share a CU and one
// hides the other's staging.  A slab is one 16-channel step when nIn <= 16 or nOut > 128.
template <bool VEC4, bool PRE>
static bool dispatch_ncb(int ncb, Metadata &m, const Table &t, const float *in, float *out, const float *w,
                         Epi epi, int n_in, int n_out, PreArgs pre, hipStream_t s) {
  const bool narrow = n_in <= 16;
#define SCN_CASE(N, NCBW, WC, GW, SSW)                                                                      \
  if (ncb <= N)                                                                                             \
    return narrow ? launch_mfma<NCBW, WC, GW, 1, VEC4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s)    \
                  : launch_mfma<NCBW, WC, GW, SSW, VEC4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
  // Levels of a few thousand sites: 64-row tiles instead of 128-row ones give the chip twice the
  // workgroups to spread (measured: 12-23 % faster at 16 k sites, 10 % at 1 k, 30 % at 250,
  // equal at 4 k, where the tap split halves in exchange).
  if (!narrow && t.n < 30000 && ncb > 8) {
    if (ncb <= 10) return launch_mfma<5, 2, 2, 1, VEC4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
    if (ncb <= 12) return launch_mfma<3, 4, 4, 1, VEC4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
    if (ncb <= 14) return launch_mfma<7, 2, 2, 1, VEC4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
    if (ncb <= 16) return launch_mfma<4, 4, 4, 1, VEC4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
  }
  SCN_CASE(1, 1, 1, 2, 2)
  SCN_CASE(2, 1, 2, 4, 2)
  SCN_CASE(4, 1, 4, 8, 2)
  SCN_CASE(6, 3, 2, 4, 2)
  SCN_CASE(8, 2, 4, 8, 2)
  SCN_CASE(10, 5, 2, 4, 1)
  SCN_CASE(12, 3, 4, 8, 1)
  SCN_CASE(14, 7, 2, 4, 1)
  SCN_CASE(16, 4, 4, 8, 1)
#undef SCN_CASE
  return false;
}

// ---- row-owner kernel for mid-width layers ----------------------------------------------
// NW wavefronts, each owning RG granules of a tile of NW*RG granules.  Only the weight slab
// goes through (double-buffered) LDS; every wavefront gathers the input rows of its own
// granules straight into A-operand registers, one (tap, slab) iteration ahead, and keeps its
// granules' [16 x nOut] accumulators in registers.  Compared with k_conv_mfma the gathered
// rows never touch LDS and one weight slab serves NW*RG*16 rows (up to 512), at the price of
// uneven MFMA work between wavefronts, which three to four wavefronts per SIMD even out.
template <int NCB, int RG, int SS, bool VEC4, int NW, bool PRE, bool BUF, bool BF16>
__global__ __launch_bounds__(NW * 64) void k_conv_rows(
    const int *__restrict__ nbr, const int *__restrict__ rowmap, int K, int64_t n, int64_t npad,
    const float *__restrict__ in, float *__restrict__ out, const float *__restrict__ wp,
    Epi epi, int n_in, int n_out, int n_slab, int tiles_per_xcd, int n_tiles,
    int n_split, float *__restrict__ partial, const float *__restrict__ pre_sc,
    const float *__restrict__ pre_sh, float pre_leak, unsigned in_bytes) {
  static_assert(!BUF || VEC4, "buffer gathers need float4 rows");
  static_assert(!BF16 || (BUF && SS % 2 == 0), "the bf16 variant: buffer gathers, steps in pairs");
  constexpr int NT = NW * 64;
  constexpr int G = NW * RG;
  constexpr int TM = G * 16;
  constexpr int WS = BF16 ? SS / 2 : SS;  // 16-byte operands per slab, column block and lane (see k_conv_mfma)
  constexpr int SLAB_F4 = WS * NCB * 64;
  constexpr int WPT = (SLAB_F4 + NT - 1) / NT;
  constexpr int SLAB_STRIDE_F4 = packed_slab_floats(SS, NCB) / (BF16 ? 8 : 4);  // as packed by k_pack_weights
  constexpr int LDS_SLAB_F4 = WPT * NT;                         // >= SLAB_STRIDE_F4 not required
  static_assert(G <= 32, "granule mask is 32 bits");
  extern __shared__ __attribute__((aligned(16))) float lds[];
  v4f *wbuf = reinterpret_cast<v4f *>(lds);                      // [2][LDS_SLAB_F4]
  int *jtab = reinterpret_cast<int *>(wbuf + 2 * LDS_SLAB_F4);   // [G][K][16]
  unsigned *gmask = reinterpret_cast<unsigned *>(jtab + G * K * 16);
  int *taplist = reinterpret_cast<int *>(gmask + K);
  int *ntaps_p = taplist + K;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, g = lane >> 4;

  const int tile = (blockIdx.x & 7) * tiles_per_xcd + (blockIdx.x >> 3);
  if (tile >= n_tiles) return;
  const int64_t tbase = (int64_t)tile * TM;

  for (int k = threadIdx.x; k < K; k += NT) gmask[k] = 0u;
  __syncthreads();
#pragma unroll
  for (int q = 0; q < RG; q++) {
    const int gr = wave * RG + q;
    const int64_t t = tbase + gr * 16 + r16;
    for (int kb = 0; kb < K; kb += 4) {
      const int k = kb + g;
      int j = -1;
      if (k < K && t < n) j = nbr[(int64_t)k * npad + t];
      if (k < K) jtab[(gr * K + k) * 16 + r16] = j;
      const unsigned long long bal = __ballot(j >= 0);
      if (lane == 0) {
#pragma unroll
        for (int gg = 0; gg < 4; gg++)
          if ((bal >> (16 * gg)) & 0xFFFFull) atomicOr(&gmask[kb + gg], 1u << gr);
      }
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int c = 0;
    for (int k = 0; k < K; k++)
      if (gmask[k] && (n_split == 1 || k % n_split == (int)blockIdx.y)) taplist[c++] = k;
    *ntaps_p = c;
  }
  __syncthreads();
  const int ntaps = *ntaps_p;
  const int total = ntaps * n_slab;

  v4f acc[RG][NCB];
#pragma unroll
  for (int q = 0; q < RG; q++)
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) acc[q][cb] = (v4f){0.f, 0.f, 0.f, 0.f};

  v4f wreg[WPT];
  v4f a_nxt[RG][SS];
  v4f a_cur[RG][WS];  // bf16: the eight values of a pair of steps
  v4f psc[SS], psh[SS];
  unsigned gm_nxt = 0, gm_cur = 0, ok_nxt = 0;
  int sl_nxt = 0;

  typedef int v4i_t __attribute__((ext_vector_type(4)));
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(in), 0, BUF ? (int)in_bytes : 0, 0x00020000);
  // COAL (see k_conv_resident): gathers are issued with the four lanes of a quad reading 64
  // consecutive bytes of one row; the values move to the MFMA's operand lanes when they are staged.
  // Only the bf16 variant, which is bound by its gathers (measured at a million sites: 64 -> 64
  // 0.46 -> 0.38 ms, 128 -> 128 0.89 -> 0.77 ms); the fp32 variant is bound by MFMA issue and
  // loses 2-6 % to the extra permutes.
  constexpr bool COAL = BUF && BF16;
  const int ld_row = COAL ? lane >> 2 : r16, ld_g = COAL ? lane & 3 : g;
  const int perm_src = (4 * r16 + g) * 4;
  auto to_operand_lanes = [&](v4f v) {
    if constexpr (COAL) {
      const float x = v.x, y = v.y, z = v.z, w = v.w;
      v.x = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(perm_src, __builtin_bit_cast(int, x)));
      v.y = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(perm_src, __builtin_bit_cast(int, y)));
      v.z = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(perm_src, __builtin_bit_cast(int, z)));
      v.w = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(perm_src, __builtin_bit_cast(int, w)));
    }
    return v;
  };
  const unsigned row_bytes = (unsigned)n_in * 4u, lane_off = 16u * (unsigned)ld_g;
  int nx_ti = 0, nx_sl = 0;  // (tap index, slab) of the next iteration to issue; issue() runs in sequence
  auto issue = [&](int) {
    const int sl = nx_sl;
    // LDS values every lane reads alike: tell the compiler, so that what follows from them
    // (weight address, branches on the granule mask) is scalar work
    const int k = __builtin_amdgcn_readfirstlane(taplist[nx_ti]);
    if (++nx_ti == ntaps) {  // slab outer, tap inner (see k_conv_mfma)
      nx_ti = 0;
      nx_sl++;
    }
    gm_nxt = __builtin_amdgcn_readfirstlane(gmask[k]);
    sl_nxt = sl;
    ok_nxt = 0;
    if (PRE) {
#pragma unroll
      for (int s = 0; s < SS; s++) {
        psc[s] = *reinterpret_cast<const v4f *>(pre_sc + (sl * SS + s) * 16 + 4 * ld_g);
        psh[s] = *reinterpret_cast<const v4f *>(pre_sh + (sl * SS + s) * 16 + 4 * ld_g);
      }
    }
    const v4f *wsrc = reinterpret_cast<const v4f *>(wp) + ((int64_t)k * n_slab + sl) * SLAB_STRIDE_F4;
#pragma unroll
    for (int i = 0; i < WPT; i++) {
      const int e = threadIdx.x + i * NT;
      wreg[i] = wsrc[e < SLAB_F4 ? e : 0];
    }
#pragma unroll
    for (int q = 0; q < RG; q++) {
      const int j = jtab[((wave * RG + q) * K + k) * 16 + ld_row];
      if constexpr (BUF) {
        // Buffer loads return zeros past the end of the buffer: an absent row becomes an
        // offset of 2 GiB (the launcher only takes this path for smaller inputs, whole slabs
        // and fewer than 2^24 rows), so no select is needed afterwards and the address is
        // one 24-bit multiply-add.
        const unsigned voff = j >= 0 ? __umul24((unsigned)j, row_bytes) + lane_off : 0x80000000u;
        if (PRE && j >= 0) ok_nxt |= 1u << q;  // zero must stay zero through the pre-activation
#pragma unroll
        for (int s = 0; s < SS; s++)
          a_nxt[q][s] = __builtin_bit_cast(
              v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, (sl * SS + s) * 64, 0));
        continue;
      }
      if (j >= 0) ok_nxt |= 1u << q;
      const float *src = in + (int64_t)(j < 0 ? 0 : j) * n_in;
#pragma unroll
      for (int s = 0; s < SS; s++) {
        const int c0 = (sl * SS + s) * 16 + 4 * g;
        if (VEC4) {
          const int cc = c0 < n_in ? c0 : n_in - 4;
          a_nxt[q][s] = *reinterpret_cast<const v4f *>(src + cc);
        } else {
          a_nxt[q][s].x = src[min(c0 + 0, n_in - 1)];
          a_nxt[q][s].y = src[min(c0 + 1, n_in - 1)];
          a_nxt[q][s].z = src[min(c0 + 2, n_in - 1)];
          a_nxt[q][s].w = src[min(c0 + 3, n_in - 1)];
        }
      }
    }
  };

  if (total > 0) issue(0);
  for (int it = 0; it < total; it++) {
    v4f *wb = wbuf + (it & 1) * LDS_SLAB_F4;
#pragma unroll
    for (int i = 0; i < WPT; i++) wb[threadIdx.x + i * NT] = wreg[i];
#pragma unroll
    for (int q = 0; q < RG; q++) {
      const bool ok = (ok_nxt >> q) & 1u;
      if constexpr (BF16) {
#pragma unroll
        for (int s = 0; s < SS; s += 2) {
          v4f v0 = a_nxt[q][s], v1 = a_nxt[q][s + 1];
          if constexpr (PRE) {
            v0 = pre_act<PRE>(v0, psc[s], psh[s], pre_leak);
            v1 = pre_act<PRE>(v1, psc[s + 1], psh[s + 1], pre_leak);
            v0 = ok ? v0 : (v4f){0.f, 0.f, 0.f, 0.f};
            v1 = ok ? v1 : (v4f){0.f, 0.f, 0.f, 0.f};
          }
          a_cur[q][s / 2] = to_operand_lanes(__builtin_bit_cast(v4f, to_bf16x8(v0, v1)));
        }
        continue;
      }
#pragma unroll
      for (int s = 0; s < SS; s++) {
        if constexpr (BUF && !PRE && !BF16) {
          a_cur[q][s] = to_operand_lanes(a_nxt[q][s]);
          continue;
        }
        if constexpr (BUF && PRE && !BF16) {
          const v4f v = pre_act<PRE>(a_nxt[q][s], psc[s], psh[s], pre_leak);
          a_cur[q][s] = to_operand_lanes(ok ? v : (v4f){0.f, 0.f, 0.f, 0.f});
          continue;
        }
        if constexpr (!BUF) {
          const int c0 = (sl_nxt * SS + s) * 16 + 4 * g;
          v4f v = pre_act<PRE>(a_nxt[q][s], psc[s], psh[s], pre_leak);
          if (VEC4) {
            if (!(ok && c0 < n_in)) v = (v4f){0.f, 0.f, 0.f, 0.f};
          } else {
            if (!(ok && c0 + 0 < n_in)) v.x = 0.f;
            if (!(ok && c0 + 1 < n_in)) v.y = 0.f;
            if (!(ok && c0 + 2 < n_in)) v.z = 0.f;
            if (!(ok && c0 + 3 < n_in)) v.w = 0.f;
          }
          a_cur[q][s] = v;
        }
      }
    }
    gm_cur = gm_nxt;
    __syncthreads();  // slab of `it` visible; every wavefront is done with the other buffer
    if (it + 1 < total) issue(it + 1);
    if (((gm_cur >> (wave * RG)) & ((1u << RG) - 1u)) == 0u) continue;  // none of my granules has the tap
#pragma unroll
    for (int s = 0; s < WS; s++) {
      v4f b[NCB];
#pragma unroll
      for (int cb = 0; cb < NCB; cb++) b[cb] = wb[(s * NCB + cb) * 64 + lane];
#pragma unroll
      for (int q = 0; q < RG; q++) {
        if (!((gm_cur >> (wave * RG + q)) & 1u)) continue;  // uniform over the wavefront
        if constexpr (BF16) {
#pragma unroll
          for (int cb = 0; cb < NCB; cb++)
            acc[q][cb] = mfma_bf16(__builtin_bit_cast(v8s, a_cur[q][s]), __builtin_bit_cast(v8s, b[cb]), acc[q][cb]);
        } else {
          const v4f av = a_cur[q][s];
#pragma unroll
          for (int cb = 0; cb < NCB; cb++) acc[q][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, b[cb].x, acc[q][cb], 0, 0, 0);
#pragma unroll
          for (int cb = 0; cb < NCB; cb++) acc[q][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, b[cb].y, acc[q][cb], 0, 0, 0);
#pragma unroll
          for (int cb = 0; cb < NCB; cb++) acc[q][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, b[cb].z, acc[q][cb], 0, 0, 0);
#pragma unroll
          for (int cb = 0; cb < NCB; cb++) acc[q][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, b[cb].w, acc[q][cb], 0, 0, 0);
        }
      }
    }
  }

  if (partial != nullptr) {  // [n_split][n_tiles * TM][NCB * 16]
    float *pt = partial + ((int64_t)blockIdx.y * n_tiles * TM + tbase) * (NCB * 16);
#pragma unroll
    for (int q = 0; q < RG; q++)
#pragma unroll
      for (int r = 0; r < 4; r++)
#pragma unroll
        for (int cb = 0; cb < NCB; cb++)
          pt[(int64_t)((wave * RG + q) * 16 + 4 * g + r) * (NCB * 16) + 16 * cb + r16] = acc[q][cb][r];
    return;
  }
  float bv[NCB], es[NCB], eh[NCB];
  const bool post = epi.sc != nullptr;
#pragma unroll
  for (int cb = 0; cb < NCB; cb++) {
    const int col = 16 * cb + r16;
    bv[cb] = (epi.bias != nullptr && col < n_out) ? epi.bias[col] : 0.0f;
    es[cb] = (post && col < n_out) ? epi.sc[col] : 1.0f;
    eh[cb] = (post && col < n_out) ? epi.sh[col] : 0.0f;
  }
#pragma unroll
  for (int q = 0; q < RG; q++) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int64_t pos = tbase + (wave * RG + q) * 16 + 4 * g + r;
      if (pos >= n) continue;
      const int64_t row = rowmap ? rowmap[pos] : pos;
      float *o = out + row * (epi.out_stride ? epi.out_stride : n_out);
#pragma unroll
      for (int cb = 0; cb < NCB; cb++) {
        const int col = 16 * cb + r16;
        float v = acc[q][cb][r] + bv[cb];
        if (post) v = epi_act(v, es[cb], eh[cb], epi.leak);
        if (col < n_out) o[col] = v;
      }
    }
  }
}

template <int NCB, int RG, int SS, bool VEC4, int NW, bool PRE, bool BUF = false, bool BF16 = false>
static bool launch_rows(Metadata &m, const Table &t, const float *in, float *out, const float *w,
                        Epi epi, int n_in, int n_out, PreArgs pre, hipStream_t s) {
  if constexpr (VEC4 && !BUF) {
    // gathers through buffer loads (no per-element selects, 32-bit addressing) when the input
    // is below 2 GiB and 2^24 rows and consists of whole slabs
    if (n_in % (16 * SS) == 0 && m.cur_in_rows > 0 && m.cur_in_rows < (1 << 24) &&
        m.cur_in_rows * n_in * 4 < ((int64_t)1 << 31) && n_in * 4 < (1 << 24)) {
      if constexpr (SS % 2 == 0) {
        if (m.bf16)
          return launch_rows<NCB, RG, SS, VEC4, NW, PRE, true, true>(m, t, in, out, w, epi, n_in, n_out, pre, s);
      }
      return launch_rows<NCB, RG, SS, VEC4, NW, PRE, true>(m, t, in, out, w, epi, n_in, n_out, pre, s);
    }
  }
  constexpr int NT = NW * 64, G = NW * RG;
  constexpr int SLAB_F4 = (BF16 ? SS / 2 : SS) * NCB * 64;
  constexpr int WPT = (SLAB_F4 + NT - 1) / NT;
  constexpr int SLAB_STRIDE = packed_slab_floats(SS, NCB);  // elements of a packed slab
  const size_t lds_bytes = (size_t)2 * WPT * NT * 16 + ((size_t)G * t.K * 16 + 2 * t.K + 4) * sizeof(int);
  if (lds_bytes > 160 * 1024) return false;
  const int cin16 = (int)ceil_div(n_in, 16);
  const int n_slab = (int)ceil_div(cin16, SS);
  const int64_t packed = (int64_t)t.K * n_slab * SLAB_STRIDE;
  float *wpack = packed_weights(m, {0, (int64_t)(uintptr_t)w, t.K, n_in, n_out, SS, NCB, BF16}, packed, [&](float *dst) {
    k_pack_weights<<<dim3((unsigned)ceil_div(packed, 256)), 256, 0, s>>>(w, dst, t.K, n_in, n_out, n_slab, SS, NCB,
                                                                        SLAB_STRIDE, take_jobs(m), BF16);
    LAUNCH_CHECK();
  });
  auto kern = k_conv_rows<NCB, RG, SS, VEC4, NW, PRE, BUF, BF16>;
  static bool attr_set = false;
  if (!attr_set) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  160 * 1024));
    attr_set = true;
  }
  const int n_tiles = (int)ceil_div(t.n, G * 16);
  const int tiles_per_xcd = (int)ceil_div(n_tiles, 8);
  int n_split = 1;
  if (n_tiles < 256) n_split = (int)std::min<int64_t>(t.K, ceil_div(512, n_tiles));
  const int64_t split_stride = (int64_t)n_tiles * G * 16 * NCB * 16;
  float *partial = scratch_partial(m, n_split, split_stride);
  kern<<<dim3((unsigned)(tiles_per_xcd * 8), n_split), NT, lds_bytes, s>>>(
      t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, in, out, wpack, epi, n_in, n_out, n_slab, tiles_per_xcd,
      n_tiles, n_split, partial, pre.sc, pre.sh, pre.leak, (unsigned)(m.cur_in_rows * n_in * 4));
  LAUNCH_CHECK();
  if (n_split > 1) {
    k_conv_reduce<<<dim3((unsigned)ceil_div(t.n * n_out, 256)), 256, 0, s>>>(partial, n_split, split_stride, NCB * 16,
                                                                          t.rowmap_ptr(), t.n, epi, out, n_out);
    LAUNCH_CHECK();
  }
  return true;
}

// ---- resident-weights kernel for narrow layers ------------------------------------------
// When the packed weights of all taps fit in LDS (K * ceil(nIn/16) * NCB KiB), a persistent
// workgroup loads them once and its wavefronts then work independently, with no barrier.
// A wavefront takes sets of RG granules and, for each set, the taps that any of its rows
// has (the OR of the table's per-granule tap masks).  The (set, tap) pairs of a wavefront
// form one stream that runs through a register pipeline four items deep: the neighbour
// indices of items i+3 and i+4 and the input rows of items i+1 and i+2 are in flight while
// item i runs its MFMAs (one item of look-ahead does not cover the latency of a gather that
// misses L2), also across the boundary between two sets, so the pipeline drains only once,
// at the wavefront's end.
// All loads are unconditional (absent rows read row 0 and are zeroed by a select; items past
// the end re-read the first set).  Granules none of whose rows has the tap skip their MFMAs.
// With accumulate != 0 the kernel adds to `out` instead of overwriting it (used to split a
// wide nIn into several launches).
template <int NCB, int RG, int SS, bool VEC4, int WAVES, bool C4, bool BUF, bool BF16>
__global__ __launch_bounds__(WAVES * 64) void k_conv_resident(
    const int *__restrict__ nbr, const int *__restrict__ rowmap, const unsigned *__restrict__ gmask, int K,
    int64_t n, int64_t npad, const float *__restrict__ in, int in_stride, float *__restrict__ out,
    const float *__restrict__ wp, Epi epi, int n_in, int n_out, int n_sets,
    int sets_per_xcd, int accumulate, int *__restrict__ queue, unsigned in_bytes, unsigned nbr_bytes) {
  static_assert(!BUF || VEC4 || C4, "buffer gathers need float4 rows or the four-channel layout");
  static_assert(!C4 || SS == 1, "the four-channel layout has one slab");
  static_assert(!BF16 || (BUF && !C4 && SS == 2), "the bf16 variant: buffer gathers, one pair of steps");
  // C4 (nIn <= 4): the MFMA's k index is the input channel itself, so a lane gathers one
  // float (row r16, channel g) and a tap costs one MFMA per column block instead of four.
  using AV = typename std::conditional<C4, float, v4f>::type;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  v4f *wl = reinterpret_cast<v4f *>(lds);  // [K][SS][NCB][64] float4, C4: [K][NCB][64] float
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int total_f4 = C4 ? K * NCB * 16 : (BF16 ? K * NCB * 64 : K * SS * NCB * 64);
  for (int e = threadIdx.x; e < total_f4; e += WAVES * 64) wl[e] = reinterpret_cast<const v4f *>(wp)[e];
  __syncthreads();  // the only barrier; every wavefront reaches it

  float bv[NCB], es[NCB], eh[NCB];
  const bool post = epi.sc != nullptr;
#pragma unroll
  for (int cb = 0; cb < NCB; cb++) {
    const int col = 16 * cb + r16;
    bv[cb] = (epi.bias != nullptr && col < n_out) ? epi.bias[col] : 0.0f;
    es[cb] = (post && col < n_out) ? epi.sc[col] : 1.0f;
    eh[cb] = (post && col < n_out) ? epi.sh[col] : 0.0f;
  }
  const int64_t n_granules = (n + 15) >> 4;
  // Tap mask of a set; a set without any rule still runs one (empty) tap so that its rows
  // get their bias.  The index is clamped: the caller decides whether the set exists.
  auto set_mask = [&](int set) {
    unsigned m = 0;
#pragma unroll
    for (int q = 0; q < RG; q++) {
      const int64_t gi = (int64_t)set * RG + q;
      m |= gmask[gi < n_granules ? gi : n_granules - 1];
    }
    return m ? m : 1u;
  };
  // One XCD (blocks b, b+8, ...) walks a contiguous range of sets.  A wavefront's first set
  // is fixed; the following ones it takes from the XCD's counter, one set ahead of the set
  // it is generating items for.  (With a fixed share per wavefront the kernel ran as long as
  // its slowest wavefront: the SIMD's arbiter favours its oldest wavefront, so the four
  // wavefronts of a SIMD finish one after the other, and shares differ in their tap counts.)
  // Every counter value is handed out once, values past the range end a wavefront's stream.
  const int xcd = blockIdx.x & 7, blk = blockIdx.x >> 3, blocks_per_xcd = gridDim.x >> 3;
  const int set_begin = xcd * sets_per_xcd;
  const int set_end = min(n_sets, set_begin + sets_per_xcd);
  const int first_round = blocks_per_xcd * WAVES;
  int *ctr = queue + xcd * 32;
  auto take = [&]() {
    int v = 0;
    if (lane == 0) v = atomicAdd(ctr, 1);
    return set_begin + first_round + __builtin_amdgcn_readfirstlane(v);
  };
  // generator of the item stream (wave-uniform state)
  int g_set = set_begin + blk * WAVES + wave;
  bool g_has = g_set < set_end;
  unsigned g_rest = g_has ? set_mask(g_set) : 0u;
  int g_next = take();           // the set after g_set
  unsigned g_mask_next = 0;      // its tap mask, read two items after g_next was requested
  int g_age = 0;
  struct Item {
    int k, set;
    bool last, valid;
  };
  auto gen = [&]() {
    if (++g_age == 2) g_mask_next = set_mask(min(g_next, n_sets - 1));
    Item it;
    it.valid = g_has;
    it.set = g_has ? g_set : 0;
    it.k = g_has ? __ffs(g_rest) - 1 : 0;
    g_rest &= g_rest - 1;
    it.last = g_has && g_rest == 0u;
    if (it.last) {
      if (g_age < 2) g_mask_next = set_mask(min(g_next, n_sets - 1));  // a set of one or two taps
      g_set = g_next;
      g_has = g_set < set_end;
      g_rest = g_mask_next;
      if (g_has) {
        g_next = take();
        g_age = 0;
      }
    }
    return it;
  };
  // Register rings, indexed by item number mod 3 (the loop below is unrolled three times so
  // that every index is a constant): neighbour indices, gathered rows, row-present bits.
  int jr[3][1];
  AV ar[3][RG][SS];
  unsigned okr[3];
  // BUF: neighbour table and input rows are read through buffer loads (32-bit offsets; an
  // offset of 2 GiB is past the end and reads as zero, which replaces the selects that zero
  // absent rows).  The launcher takes this variant when both buffers are below 2 GiB, the rows
  // fewer than 2^24 and the channel part a whole number of slabs.
  const __amdgpu_buffer_rsrc_t in_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(in), 0, BUF ? (int)in_bytes : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t nbr_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<int *>(nbr), 0, BUF ? (int)nbr_bytes : 0, 0x00020000);
  const unsigned row_bytes = (unsigned)in_stride * 4u;
  const unsigned lane_off = C4 ? (g < n_in ? 4u * (unsigned)g : 0x80000000u) : 16u * (unsigned)g;
  // One load fetches the indices of the whole set (lane l: row l of the set); issue_a hands
  // each lane the index of its own row of every granule through a lane permute, which costs an
  // LDS-crossbar instruction instead of a memory instruction per granule.
  const int set_lane = lane % (RG * 16);
  auto issue_j = [&](const Item &it, int *j) {
    if constexpr (BUF) {
      const unsigned t = min((unsigned)it.set * (RG * 16) + set_lane, (unsigned)(n - 1));
      j[0] = __builtin_amdgcn_raw_buffer_load_b32(nbr_rsrc, t * 4u, (unsigned)it.k * (unsigned)npad * 4u, 0);
    } else {
      const int64_t t = min((int64_t)it.set * (RG * 16) + set_lane, n - 1);
      j[0] = nbr[(int64_t)it.k * npad + t];
    }
  };
  // COAL: a gather instruction reads 16 rows x 64 bytes.  In the MFMA's operand layout (lane
  // g * 16 + r: bytes [16 g, 16 g + 16) of row r) neighbouring lanes read different rows, 64
  // separate accesses for the texture unit; read as lane 4 r + g instead, the four lanes of a
  // quad read 64 consecutive bytes, one access, and the values change lanes afterwards (an
  // LDS-crossbar permute per register, at use).
  constexpr bool COAL = BUF && VEC4 && !C4;
  const int ld_row = COAL ? lane >> 2 : r16;                 // row of a granule this lane loads
  const unsigned ld_off = COAL ? 16u * (unsigned)(lane & 3) : lane_off;
  const int perm_src = (4 * r16 + g) * 4;                    // byte address of the lane that loaded this lane's operand
  auto to_operand_lanes = [&](v4f v) {
    if constexpr (COAL) {
      const float x = v.x, y = v.y, z = v.z, w = v.w;  // (element references do not survive a bit cast)
      v.x = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(perm_src, __builtin_bit_cast(int, x)));
      v.y = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(perm_src, __builtin_bit_cast(int, y)));
      v.z = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(perm_src, __builtin_bit_cast(int, z)));
      v.w = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(perm_src, __builtin_bit_cast(int, w)));
    }
    return v;
  };
  auto issue_a = [&](const Item &it, const int *jset, AV (*a)[SS], unsigned &okbits) {
    okbits = 0;
    int j[RG];
#pragma unroll
    for (int q = 0; q < RG; q++) j[q] = __shfl(jset[0], q * 16 + ld_row, 64);
#pragma unroll
    for (int q = 0; q < RG; q++) {
      const bool ok = j[q] >= 0 && (int64_t)it.set * (RG * 16) + q * 16 + ld_row < n;
      okbits |= ok ? 1u << q : 0u;
      if constexpr (BUF) {
        const unsigned voff = ok ? (__umul24((unsigned)j[q], row_bytes) + ld_off) : 0x80000000u;
#pragma unroll
        for (int s = 0; s < SS; s++) {
          if constexpr (C4)
            a[q][s] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(in_rsrc, voff, 0, 0));
          else
            a[q][s] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(in_rsrc, voff, s * 64, 0));
        }
        continue;
      }
      const float *src = in + (int64_t)(ok ? j[q] : 0) * in_stride;
#pragma unroll
      for (int s = 0; s < SS; s++) {
        const int c0 = s * 16 + 4 * g;
        if constexpr (C4) {
          a[q][s] = src[min(g, n_in - 1)];
        } else if constexpr (VEC4) {
          const int cc = c0 < n_in ? c0 : n_in - 4;
          a[q][s] = *reinterpret_cast<const v4f *>(src + cc);
        } else {
          a[q][s].x = src[min(c0 + 0, n_in - 1)];
          a[q][s].y = src[min(c0 + 1, n_in - 1)];
          a[q][s].z = src[min(c0 + 2, n_in - 1)];
          a[q][s].w = src[min(c0 + 3, n_in - 1)];
        }
      }
    }
  };

  v4f acc[RG][NCB];
#pragma unroll
  for (int q = 0; q < RG; q++)
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) acc[q][cb] = (v4f){0.f, 0.f, 0.f, 0.f};

  // Items in flight: I0 runs its MFMAs now, I1's rows are on their way, I2's indices have
  // arrived (its rows are requested next), I3's indices are on their way.
  Item I0 = gen(), I1 = gen(), I2 = gen(), I3 = gen();
  issue_j(I0, jr[0]);
  issue_j(I1, jr[1]);
  issue_a(I0, jr[0], ar[0], okr[0]);
  issue_j(I2, jr[2]);
  issue_a(I1, jr[1], ar[1], okr[1]);
  issue_j(I3, jr[0]);

  auto step = [&](auto slot) {
    constexpr int S = decltype(slot)::value, S1 = (S + 1) % 3, S2 = (S + 2) % 3;
    issue_a(I2, jr[S2], ar[S2], okr[S2]);
    const Item I4 = gen();
    issue_j(I4, jr[S1]);

    const int64_t t0 = (int64_t)I0.set * (RG * 16);
    const int k_cur = I0.k;
    const unsigned okb = okr[S];
    if (__ballot(okb != 0u) != 0ull) {
      if constexpr (C4) {
        float b[NCB];
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) b[cb] = lds[(k_cur * NCB + cb) * 64 + lane];
#pragma unroll
        for (int q = 0; q < RG; q++) {
          const bool ok = (okb >> q) & 1u;
          if (__ballot(ok) == 0ull) continue;  // uniform: no row of this granule has the tap
          const float av = BUF ? ar[S][q][0] : ((ok && g < n_in) ? ar[S][q][0] : 0.f);
#pragma unroll
          for (int cb = 0; cb < NCB; cb++) acc[q][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, b[cb], acc[q][cb], 0, 0, 0);
        }
      } else if constexpr (BF16) {
        // one operand per column block holds both steps (bf16); the gathered rows are rounded here
        v4f b[NCB];
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) b[cb] = wl[(k_cur * NCB + cb) * 64 + lane];
#pragma unroll
        for (int q = 0; q < RG; q++) {
          const bool ok = (okb >> q) & 1u;
          if (__ballot(ok) == 0ull) continue;  // uniform: no row of this granule has the tap
          v8s av = to_bf16x8(ar[S][q][0], ar[S][q][1]);
          if constexpr (COAL) av = __builtin_bit_cast(v8s, to_operand_lanes(__builtin_bit_cast(v4f, av)));
#pragma unroll
          for (int cb = 0; cb < NCB; cb++) acc[q][cb] = mfma_bf16(av, __builtin_bit_cast(v8s, b[cb]), acc[q][cb]);
        }
      } else {
        v4f b[SS][NCB];
#pragma unroll
        for (int s = 0; s < SS; s++)
#pragma unroll
          for (int cb = 0; cb < NCB; cb++) b[s][cb] = wl[((k_cur * SS + s) * NCB + cb) * 64 + lane];
#pragma unroll
        for (int q = 0; q < RG; q++) {
          const bool ok = (okb >> q) & 1u;
          if (__ballot(ok) == 0ull) continue;  // uniform: no row of this granule has the tap
#pragma unroll
          for (int s = 0; s < SS; s++) {
            const int c0 = s * 16 + 4 * g;
            v4f av = to_operand_lanes(ar[S][q][s]);
            if (BUF) {
            } else if (VEC4) {
              if (!(ok && c0 < n_in)) av = (v4f){0.f, 0.f, 0.f, 0.f};
            } else {
              if (!(ok && c0 + 0 < n_in)) av.x = 0.f;
              if (!(ok && c0 + 1 < n_in)) av.y = 0.f;
              if (!(ok && c0 + 2 < n_in)) av.z = 0.f;
              if (!(ok && c0 + 3 < n_in)) av.w = 0.f;
            }
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) acc[q][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, b[s][cb].x, acc[q][cb], 0, 0, 0);
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) acc[q][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, b[s][cb].y, acc[q][cb], 0, 0, 0);
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) acc[q][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, b[s][cb].z, acc[q][cb], 0, 0, 0);
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) acc[q][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, b[s][cb].w, acc[q][cb], 0, 0, 0);
          }
        }
      }
    }
    if (I0.last) {  // the set is complete: write its rows, start the next set from zero
#pragma unroll
      for (int q = 0; q < RG; q++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int64_t pos = t0 + q * 16 + 4 * g + r;
          if (pos < n) {
            const int64_t row = rowmap ? rowmap[pos] : pos;
            float *o = out + row * n_out;
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) {
              const int col = 16 * cb + r16;
              if (col < n_out) {
                float v = acc[q][cb][r] + (accumulate ? o[col] : bv[cb]);
                if (post) v = epi_act(v, es[cb], eh[cb], epi.leak);
                o[col] = v;
              }
            }
          }
        }
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) acc[q][cb] = (v4f){0.f, 0.f, 0.f, 0.f};
      }
    }
    I0 = I1;
    I1 = I2;
    I2 = I3;
    I3 = I4;
  };
  while (true) {  // items after the last valid one are invalid: every wavefront leaves here
    if (!I0.valid) break;
    step(std::integral_constant<int, 0>{});
    if (!I0.valid) break;
    step(std::integral_constant<int, 1>{});
    if (!I0.valid) break;
    step(std::integral_constant<int, 2>{});
  }
  // The last workgroup to get here leaves the counters at zero for the next launch (every
  // workgroup has taken its last set by now: nobody adds to them any more).
  __syncthreads();
  if (threadIdx.x == 0) {
    __threadfence();
    if (atomicAdd(queue + 8 * 32, 1) == (int)gridDim.x - 1) {
      for (int i = 0; i < 9; i++) queue[i * 32] = 0;
    }
  }
}

// B operands of the four-channel layout: wp[(k * NCB + cb) * 64 + lane] = w[k][lane / 16][16 cb + lane % 16].
// Also clears the set counters, as k_pack_weights_part does.
__global__ void k_pack_weights_c4(const float *w, float *wp, int K, int n_in, int n_out, int NCB, int *queue,
                                  CoefJobs jobs) {
  coef_jobs(jobs);
  if (blockIdx.x == 0 && threadIdx.x < 8) queue[threadIdx.x * 32] = 0;
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= K * NCB * 64) return;
  const int lane = i & 63, cb = (i >> 6) % NCB, k = i / (64 * NCB);
  const int ch = lane >> 4, col = 16 * cb + (lane & 15);
  wp[i] = (ch < n_in && col < n_out) ? w[((int64_t)k * n_in + ch) * n_out + col] : 0.0f;
}

template <int NCB, int RG, int SS, bool VEC4, int WAVES, bool C4, bool BUF = false, bool BF16 = false>
static void launch_resident_kernel(Metadata &m, const Table &t, const float *in, int in_stride, float *out,
                                   const float *wpack, Epi epi, int n_in_part, int n_out, int accumulate,
                                   size_t lds_bytes, int per_cu, hipStream_t s) {
  // bytes from `in` (which may point at a channel offset inside the first row) to the end
  const int64_t in_bytes = (m.cur_in_rows * in_stride - (in - m.cur_in_base)) * 4;
  const int64_t nbr_bytes = (int64_t)t.K * t.npad * 4;
  if constexpr ((VEC4 || C4) && !BUF) {
    const bool whole = C4 || n_in_part == 16 * SS;
    if (whole && m.cur_in_rows > 0 && m.cur_in_rows < (1 << 24) && in_stride * 4 < (1 << 24) && in_bytes > 0 &&
        in_bytes < ((int64_t)1 << 31) && nbr_bytes < ((int64_t)1 << 31)) {
      launch_resident_kernel<NCB, RG, SS, VEC4, WAVES, C4, true, BF16>(m, t, in, in_stride, out, wpack, epi, n_in_part,
                                                                       n_out, accumulate, lds_bytes, per_cu, s);
      return;
    }
  }
  if constexpr (BF16 && !BUF) {
    throw Error("internal: the bf16 resident kernel needs buffer gathers");
  } else {
  auto kern = k_conv_resident<NCB, RG, SS, VEC4, WAVES, C4, BUF, BF16>;
  static bool attr_set = false;
  if (!attr_set) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  160 * 1024));
    attr_set = true;
  }
  const int n_sets = (int)ceil_div(t.n, RG * 16);
  const int sets_per_xcd = (int)ceil_div(n_sets, 8);
  const int blocks = 8 * (int)std::max<int64_t>(1, std::min<int64_t>(32 * per_cu, ceil_div(sets_per_xcd, WAVES)));
  kern<<<dim3(blocks), WAVES * 64, lds_bytes, s>>>(t.nbr.p, t.rowmap_ptr(), t.gmask.p, t.K, t.n, t.npad, in, in_stride,
                                                   out, wpack, epi, n_in_part, n_out, n_sets, sets_per_xcd,
                                                   accumulate, scratch_queue(m, s), (unsigned)in_bytes, (unsigned)nbr_bytes);
  LAUNCH_CHECK();
  }
}

// Whether launch_resident_kernel would take its buffer-gather variant for this input.
static bool resident_buffer_gathers(const Metadata &m, const Table &t, const float *in, int in_stride) {
  const int64_t in_bytes = (m.cur_in_rows * in_stride - (in - m.cur_in_base)) * 4;
  const int64_t nbr_bytes = (int64_t)t.K * t.npad * 4;
  return m.cur_in_rows > 0 && m.cur_in_rows < (1 << 24) && in_stride * 4 < (1 << 24) && in_bytes > 0 &&
         in_bytes < ((int64_t)1 << 31) && nbr_bytes < ((int64_t)1 << 31);
}

// One launch over channels [c_lo, c_lo + n_in_part) of the input rows.
template <int NCB, int SS, bool VEC4>
static void launch_resident_part(Metadata &m, const Table &t, const float *in, int in_stride, float *out,
                                 const float *w, int w_in_stride_rows, Epi epi, int n_in_part,
                                 int n_out, int accumulate, hipStream_t s) {
  constexpr int RG = 2;  // 32 rows per set: measured faster than 64 (more wavefronts in flight)
  const int64_t packed = (int64_t)t.K * SS * NCB * 256;
  int *queue = scratch_queue(m, s);
  bool bf16 = false;
  if constexpr (SS == 2 && VEC4)  // bf16 operands (when asked for): a whole 32-channel part, buffer gathers
    bf16 = m.bf16 && n_in_part == 32 && resident_buffer_gathers(m, t, in, in_stride);
  // weights of this channel range: rows [c_lo, c_lo + n_in_part) of every tap's [nIn x nOut] slice
  const float *wpack = packed_weights(m, {1, (int64_t)(uintptr_t)w, t.K, w_in_stride_rows, n_in_part, n_out, SS, NCB, bf16},
                                      packed, [&](float *dst) {
    k_pack_weights_part<<<dim3((unsigned)ceil_div(packed, 256)), 256, 0, s>>>(w, dst, t.K, w_in_stride_rows, n_in_part,
                                                                             n_out, SS, NCB, queue, take_jobs(m), bf16);
    LAUNCH_CHECK();
  });
  if constexpr (SS == 2 && VEC4) {
    if (bf16) {
      const size_t lds16 = (size_t)packed * 2;  // 2-byte elements
      const int per_cu16 = (int)std::max<size_t>(1, std::min<size_t>(4, (160 * 1024) / lds16));
      if (lds16 > 80 * 1024)
        launch_resident_kernel<NCB, RG, SS, VEC4, 16, false, true, true>(m, t, in, in_stride, out, wpack, epi, n_in_part,
                                                                         n_out, accumulate, lds16, 1, s);
      else
        launch_resident_kernel<NCB, RG, SS, VEC4, 8, false, true, true>(m, t, in, in_stride, out, wpack, epi, n_in_part,
                                                                        n_out, accumulate, lds16, per_cu16, s);
      return;
    }
  }
  const size_t lds_bytes = (size_t)packed * sizeof(float);
  if (lds_bytes > 80 * 1024) {
    launch_resident_kernel<NCB, RG, SS, VEC4, 16, false>(m, t, in, in_stride, out, wpack, epi, n_in_part, n_out,
                                                         accumulate, lds_bytes, 1, s);
  } else {
    const int per_cu = (int)std::max<size_t>(1, std::min<size_t>(4, (160 * 1024) / std::max<size_t>(lds_bytes, 1)));
    launch_resident_kernel<NCB, RG, SS, VEC4, 8, false>(m, t, in, in_stride, out, wpack, epi, n_in_part, n_out,
                                                        accumulate, lds_bytes, per_cu, s);
  }
}

// nIn <= 4 (the first layer of most networks): four-channel layout, 64 rows per set.
template <int NCB>
static void launch_resident_c4(Metadata &m, const Table &t, const float *in, float *out, const float *w,
                               Epi epi, int n_in, int n_out, hipStream_t s) {
  if (in == m.cur_in_base && conv_first_serves(t, m.cur_in_rows, n_in, n_out)) {
    // epi.sc / epi.sh point at arrays nobody fills on this path: the kernel folds the batch norm itself
    take_jobs(m);
    conv_first_forward(t, in, m.cur_in_rows, out, w, epi.bias, m.post_raw, epi.leak, n_in, n_out, s);
    return;
  }
  const int packed = t.K * NCB * 64;
  int *queue = scratch_queue(m, s);
  const float *wpack = packed_weights(m, {2, (int64_t)(uintptr_t)w, t.K, n_in, n_out, NCB}, packed, [&](float *dst) {
    k_pack_weights_c4<<<dim3((unsigned)ceil_div(packed, 256)), 256, 0, s>>>(w, dst, t.K, n_in, n_out, NCB, queue,
                                                                          take_jobs(m));
    LAUNCH_CHECK();
  });
  launch_resident_kernel<NCB, 4, 1, false, 8, true>(m, t, in, n_in, out, wpack, epi, n_in, n_out, 0,
                                                    (size_t)packed * sizeof(float), 3, s);
}

// Narrow layers: nOut <= 32, any nIn, K <= 32.  nIn is processed in parts of up to 32
// channels so that every part's weights fit in LDS; parts after the first accumulate.
// The resident kernel serves nOut <= 32 with up to 32 taps.  It takes the input channels in
// parts of 32 (every part after the first re-reads and re-writes the output) and has no fused
// batch norm, so from 64 input channels on the row-owner kernel is faster (measured).
static bool resident_fits(const Metadata &m, const Table &t, int n_in, int n_out, bool with_bn) {
  if (!(t.K <= 32 && n_out <= 32 && t.gmask.p != nullptr)) return false;
  // the resident kernel computes in fp32 only; from two parts on the row-owner kernel's bf16
  // variant is faster (measured)
  if (m.bf16 && n_in >= 64 && n_in % 32 == 0) return false;
  // several parts re-read and re-write the output once per part: with few taps (strided and
  // transposed convolutions) that costs more than the convolution itself
  if (n_in > 32 && t.K <= 8) return false;
  (void)with_bn;
  return n_in < 64;  // two parts and more: the row-owner kernel is 3 % (64 -> 32) to 10 % (96 -> 32) faster at 1 M sites
}

// No fused batch norm here: this kernel's time goes into the vector instructions around its
// small MFMA blocks, and normalising every gathered value (each row is gathered once per tap
// that reaches it) costs more than one extra pass over the rows.
static bool try_resident(Metadata &m, const Table &t, const float *in, float *out, const float *w,
                         Epi epi, int n_in, int n_out, hipStream_t s) {
  if (!resident_fits(m, t, n_in, n_out, false)) return false;
  const bool vec4 = n_in % 4 == 0 && ((uintptr_t)in % 16 == 0);
  const int ncb = (int)ceil_div(n_out, 16);
  if (n_in <= 4) {
    if (ncb == 1) launch_resident_c4<1>(m, t, in, out, w, epi, n_in, n_out, s);
    else launch_resident_c4<2>(m, t, in, out, w, epi, n_in, n_out, s);
    return true;
  }
  for (int c_lo = 0; c_lo < n_in; c_lo += 32) {
    const int part = std::min(32, n_in - c_lo);
    const float *in_p = in + c_lo;
    const float *w_p = w + (int64_t)c_lo * n_out;
    const int acc = c_lo > 0;
    Epi b;  // bias with the first part, the following layer's batch norm with the last
    if (!acc) b.bias = epi.bias;
    if (c_lo + 32 >= n_in) {
      b.sc = epi.sc;
      b.sh = epi.sh;
      b.leak = epi.leak;
    }
#define SCN_RES(NCBV, SSV)                                                                                   \
  do {                                                                                                       \
    if (vec4)                                                                                                \
      launch_resident_part<NCBV, SSV, true>(m, t, in_p, n_in, out, w_p, n_in, b, part, n_out, acc, s);       \
    else                                                                                                     \
      launch_resident_part<NCBV, SSV, false>(m, t, in_p, n_in, out, w_p, n_in, b, part, n_out, acc, s);      \
  } while (0)
    if (ncb == 1 && part <= 16) SCN_RES(1, 1);
    else if (ncb == 1) SCN_RES(1, 2);
    else if (part <= 16) SCN_RES(2, 1);
    else SCN_RES(2, 2);
#undef SCN_RES
  }
  return true;
}

// Mid-width layers (32 < nOut <= 128): row-owner kernel with 128- or 64-row workgroups (measured
// best on room scenes: small workgroups, five or more per CU, even out the work between
// barriers better than 256- or 512-row ones).  Above 128 outputs the accumulators of a
// granule no longer leave room for this layout's operands and k_conv_mfma is as fast.
template <bool VEC4, bool PRE>
static bool dispatch_rows(Metadata &m, const Table &t, const float *in, float *out, const float *w,
                          Epi epi, int n_in, int n_out, PreArgs pre, hipStream_t s) {
  const int ncb = (int)ceil_div(n_out, 16);
  const bool narrow = n_in <= 16;
  // 64-row workgroups where 128-row ones would leave a CU with one or two of them (a level of
  // 60 k sites is 480 such workgroups for 256 CUs: one wavefront per SIMD, nothing to run while
  // it waits for its gathers).  Measured: 13-18 % faster at 62 k sites, 5 % at 15 k and 250 k,
  // equal at 1 M except for 64 output planes, which gain 2 % there too.
  if (!narrow && ncb > 2 && (t.n < 300000 || ncb <= 4)) {
    if (ncb <= 4) return launch_rows<4, 1, 2, VEC4, 4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
    if (ncb <= 6) return launch_rows<6, 1, 2, VEC4, 4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
    if (ncb <= 8) return launch_rows<8, 1, 2, VEC4, 4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
  }
  if (ncb <= 2)
    return narrow ? launch_rows<2, 2, 1, VEC4, 4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s)
                  : launch_rows<2, 2, 2, VEC4, 4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
  if (ncb <= 4) return launch_rows<4, 2, 1, VEC4, 4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);  // narrow
  if (ncb <= 6)
    return narrow ? launch_rows<6, 2, 1, VEC4, 4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s)
                  : launch_rows<6, 2, 2, VEC4, 4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
  if (ncb <= 8)
    return narrow ? launch_rows<8, 1, 1, VEC4, 8, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s)
                  : launch_rows<8, 1, 2, VEC4, 8, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
  return false;
}

template <bool PRE>
static bool conv_mfma_paths(Metadata &m, const Table &t, const float *in, float *out, const float *w,
                            Epi epi, int n_in, int n_out, PreArgs pre, hipStream_t s) {
  if (!PRE && try_resident(m, t, in, out, w, epi, n_in, n_out, s)) return true;
  const bool vec4 = n_in % 4 == 0 && ((uintptr_t)in % 16 == 0);
  if (n_out <= 128 && t.K <= 1024) {
    if (vec4 ? dispatch_rows<true, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s)
             : dispatch_rows<false, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s))
      return true;
  }
  if (t.K <= 1024) {
    const int ncb = (int)ceil_div(n_out, 16);
    if (vec4 ? dispatch_ncb<true, PRE>(ncb, m, t, in, out, w, epi, n_in, n_out, pre, s)
             : dispatch_ncb<false, PRE>(ncb, m, t, in, out, w, epi, n_in, n_out, pre, s))
      return true;
  }
  return false;
}

// dst[r][c] = w[r][c0 + c], c < wc: one column range of a [rows x n_out] weight matrix, contiguous.
__global__ void k_take_columns(const float *w, int64_t rows, int n_out, int c0, int wc, float *dst) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * wc) return;
  const int64_t r = i / wc;
  const int c = (int)(i - r * wc);
  dst[i] = w[r * n_out + c0 + c];
}

// bn: optional eval batch norm + leaky ReLU applied to the input rows before the convolution
// (what a BatchNormalization module in front of the convolution computes), fused into the
// gather; post: the same for a BatchNormalization module behind the convolution, applied to
// the output values as they are stored.  nullptr for a plain convolution.
void conv_forward(Metadata &m, const Table &t, const float *in, int64_t n_in_rows, float *out, const float *w,
                  const float *bias, int n_in, int n_out, int groups, const BnArgs *bn, const BnArgs *post,
                  hipStream_t s) {
  struct FrozenReset {  // a frozen set serves one call
    Metadata &m;
    ~FrozenReset() { m.frozen = nullptr; }
  } frozen_reset{m};
  if (groups < 1 || n_in < 1 || n_out < 1 || n_in % groups || n_out % groups)
    throw Error("channel counts must be positive multiples of groups");
  if (t.n == 0) return;
  if (m.fixed_scratch && (bn || post || groups != 1))
    throw Error("allocation-free convolution: plain convolutions with groups = 1 only");
  Epi epi;
  epi.bias = bias;
  m.jobs = CoefJobs();
  m.cur_in_rows = n_in_rows;
  m.cur_in_base = in;
  FrozenParams *frozen = m.fixed_scratch ? nullptr : m.frozen;
  m.post_raw = CoefJob();
  if (post) {
    DevBuf<float> &buf = frozen ? frozen->post : m.postbuf;
    buf.reserve(2 * (size_t)n_out);
    m.jobs.post = CoefJob{post->mean, post->var, post->gamma, post->beta, post->eps, n_out, n_out, buf.p, buf.p + n_out};
    m.post_raw = m.jobs.post;
    epi.sc = buf.p;
    epi.sh = buf.p + n_out;
    epi.leak = post->leak;
  }
  const bool pre_fused = bn && groups == 1 && !resident_fits(m, t, n_in, n_out, true);
  PreArgs pre;
  if (pre_fused) {
    const int n_pad = (int)round_up(n_in, 64) + 64;
    DevBuf<float> &buf = frozen ? frozen->pre : m.prebuf;
    buf.reserve(2 * (size_t)n_pad);
    m.jobs.pre = CoefJob{bn->mean, bn->var, bn->gamma, bn->beta, bn->eps, n_in, n_pad, buf.p, buf.p + n_pad};
    pre.sc = buf.p;
    pre.sh = buf.p + n_pad;
    pre.leak = bn->leak;
  }
  if (frozen) {
    // folded once, by a launch of their own (the packing launches that normally fold them on the
    // side do not run when the packed weights are found)
    if (frozen->post_done) m.jobs.post = CoefJob();
    if (frozen->pre_done) m.jobs.pre = CoefJob();
    if (m.jobs.post.n_pad || m.jobs.pre.n_pad) {
      k_coefs<<<dim3(1), 256, 0, s>>>(take_jobs(m));
      LAUNCH_CHECK();
    }
    frozen->post_done = frozen->post_done || post != nullptr;
    frozen->pre_done = frozen->pre_done || pre_fused;
  }
  if (pre_fused) {
    if (conv_mfma_paths<true>(m, t, in, out, w, epi, n_in, n_out, pre, s)) return;
    m.jobs.pre = CoefJob();
  }
  const float *src = in;
  if (bn) {  // no fused kernel for this shape: normalise the rows in a pass of their own
    m.bntmp.reserve((size_t)std::max<int64_t>(n_in_rows, 1) * n_in);
    bn_eval_forward(in, m.bntmp.p, n_in_rows, n_in, n_in, n_in, bn->mean, bn->var, bn->gamma, bn->beta, bn->eps,
                    bn->leak, s);
    src = m.bntmp.p;
    m.cur_in_base = src;
  }
  if (groups == 1 && conv_mfma_paths<false>(m, t, src, out, w, epi, n_in, n_out, PreArgs(), s)) return;
  if (groups == 1 && n_out > 256 && t.n > 0) {
    // More output planes than the MFMA kernels hold accumulators for (the input gradient of a
    // convolution behind a JoinTable is one): ranges of at most 256 columns, each a convolution
    // of its own over that range's weights, written into its columns of `out`.
    const int ranges = (int)ceil_div(n_out, 256);
    const int width = (int)round_up(ceil_div(n_out, ranges), 16);
    const int64_t rows_w = (int64_t)t.K * n_in;
    m.wcols.reserve((size_t)rows_w * n_out);
    bool ok = true;
    for (int c0 = 0; c0 < n_out && ok; c0 += width) {
      const int wc = std::min(width, n_out - c0);
      float *dst = m.wcols.p + rows_w * c0;
      k_take_columns<<<dim3((unsigned)ceil_div(rows_w * wc, 256)), 256, 0, s>>>(w, rows_w, n_out, c0, wc, dst);
      LAUNCH_CHECK();
      Epi e = epi;
      if (e.bias) e.bias += c0;
      if (e.sc) e.sc += c0, e.sh += c0;
      e.out_stride = n_out;
      ok = conv_mfma_paths<false>(m, t, src, out + c0, dst, e, n_in, wc, PreArgs(), s);
    }
    if (ok) return;
  }
  if (m.jobs.post.n_pad) {  // no packing launch on this path: fold the coefficients by themselves
    k_coefs<<<dim3(1), 256, 0, s>>>(take_jobs(m));
    LAUNCH_CHECK();
  }
  int64_t total = t.n * n_out;
  k_conv_generic<<<dim3((unsigned)ceil_div(total, 256)), 256, 0, s>>>(t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, src,
                                                                       out, w, epi, n_in, n_out, groups);
  LAUNCH_CHECK();
}

}  // namespace scn
