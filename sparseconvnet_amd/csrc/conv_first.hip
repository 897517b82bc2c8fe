// Convolution forward for the first layer of a network: nIn <= 4, nOut <= 32, up to 32 taps
// (CPU/Convolution.cpp:45-79,117-150 with the few input planes an input layer hands over).
//
// With so few input planes the layer is bound by how many separate memory accesses its gathers
// make, not by arithmetic, so the matrix instruction is fed differently from the wider
// kernels: the contraction index of v_mfma_f32_16x16x4_f32 is the filter TAP (four taps per
// instruction), and each input plane gets an instruction of its own.  Lane (g, r16) then
// gathers the WHOLE input row (nIn consecutive floats, one access) that tap g of the group
// needs for row r16 of a granule, where a channel-per-lane layout makes nIn single-float
// accesses of it; and no lanes idle on a fourth channel that does not exist.
//
// One wavefront owns a set of 64 positions (four granules).  The taps that any row of the
// set has (OR of the granules' tap masks) are taken four at a time; per group of four:
//   indices   lane (g, r16) loads nbr[tap_g][position] for each granule (one load, four
//             64-byte runs); a group's unused lanes (tap count not a multiple of four) point
//             past the table, read 0 and are turned into "absent",
//   gather    one buffer load of nIn floats per granule; an absent neighbour is an offset past
//             the end of the buffer and reads as zeros,
//   weights   B operand of (plane c, column block cb): lane (g, r16) reads
//             w[tap_g][c][16 cb + r16] from the copy of all weights in LDS,
//   MFMAs     nIn x NCB per granule that has one of the group's taps.
// The group loop is software-pipelined two deep (the next group's gathers and the indices of
// the one after are in flight during a group's MFMAs); all its loads are unconditional so that
// the compiler can count them, groups past the end read nothing (offsets past the end).
// Outputs leave through buffer stores: rows past n and columns past nOut are dropped by
// range checking.  Workgroups b, b + 8, ... (one XCD) take a contiguous range of sets.
#include "metadata.h"

namespace scn {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v3f __attribute__((ext_vector_type(3)));
typedef float v2f __attribute__((ext_vector_type(2)));

// floats per tap of the weights in LDS: [c][cb][16], padded so that two taps an odd number
// apart start 16 banks apart
constexpr int first_tap_floats(int n_in, int ncb) {
  return (n_in * ncb * 16) % 32 == 0 ? n_in * ncb * 16 + 16 : n_in * ncb * 16;
}

template <int NIN> struct RowOf;
template <> struct RowOf<1> { typedef float type; };
template <> struct RowOf<2> { typedef v2f type; };
template <> struct RowOf<3> { typedef v3f type; };
template <> struct RowOf<4> { typedef v4f type; };

template <int NIN>
__device__ inline typename RowOf<NIN>::type load_row(__amdgpu_buffer_rsrc_t rsrc, unsigned voff) {
  if constexpr (NIN == 1)
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voff, 0, 0));
  else if constexpr (NIN == 2)
    return __builtin_bit_cast(v2f, __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff, 0, 0));
  else if constexpr (NIN == 3)
    return __builtin_bit_cast(v3f, __builtin_amdgcn_raw_buffer_load_b96(rsrc, voff, 0, 0));
  else
    return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, 0, 0));
}
template <int NIN> __device__ inline float plane_of(const typename RowOf<NIN>::type &v, int c) {
  if constexpr (NIN == 1) return v;
  else return v[c];
}

template <int NIN, int NCB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 5))) void k_conv_first(
    const int *__restrict__ nbr, const int *__restrict__ rowmap, const unsigned *__restrict__ gmask, int K,
    int64_t n, int64_t npad, const float *__restrict__ in, float *__restrict__ out,
    const float *__restrict__ w, const float *__restrict__ bias, CoefJob bn, float leak, int n_out, int n_sets,
    int sets_per_xcd, int sets_per_wave, unsigned in_bytes, unsigned nbr_bytes, unsigned out_bytes) {
  typedef typename RowOf<NIN>::type Row;
  constexpr int WS = first_tap_floats(NIN, NCB);
  // wl[k][c][cb][j] = w[k][c][16 cb + j]; tap K (what a group's unused slots read) is zero
  extern __shared__ __attribute__((aligned(16))) float wl[];  // [(K + 1)][WS]
  for (int e = threadIdx.x; e < (K + 1) * WS; e += 256) {
    const int k = e / WS, r = e - k * WS;
    const int c = r / (NCB * 16), col = 16 * ((r / 16) % NCB) + (r & 15);
    wl[e] = (k < K && c < NIN && col < n_out) ? w[((int64_t)k * NIN + c) * n_out + col] : 0.0f;
  }
  __syncthreads();  // the only barrier
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  // bn: the batch norm + leaky ReLU of the layer behind, folded to scale / shift per output
  // column here (the wider kernels have their weight-packing launch do it)
  const bool post = bn.n > 0;
  float bv[NCB], es[NCB], eh[NCB];
  unsigned col_off[NCB];
#pragma unroll
  for (int cb = 0; cb < NCB; cb++) {
    const int col = 16 * cb + r16;
    bv[cb] = (bias != nullptr && col < n_out) ? bias[col] : 0.0f;
    es[cb] = 1.0f;
    eh[cb] = 0.0f;
    if (post && col < n_out) {
      es[cb] = (1.0f / sqrtf(bn.var[col] + bn.eps)) * (bn.gamma ? bn.gamma[col] : 1.0f);
      eh[cb] = -bn.mean[col] * es[cb] + (bn.beta ? bn.beta[col] : 0.0f);
    }
    col_off[cb] = 4u * (unsigned)col;
  }
  const __amdgpu_buffer_rsrc_t in_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(in), 0, (int)in_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t nbr_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<int *>(nbr), 0, (int)nbr_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(out, 0, (int)out_bytes, 0x00020000);
  constexpr int ROW_BYTES = NIN * 4;
  const unsigned out_row_bytes = (unsigned)n_out * 4u;
  const unsigned tap_stride = (unsigned)npad * 4u;
  const unsigned shift8 = 8u * (unsigned)g;
  const int64_t n_granules = (n + 15) >> 4;
  const int xcd = blockIdx.x & 7, blk = blockIdx.x >> 3;
  // sets_per_xcd == 0 (the table's positions are pattern-sorted as a whole, most expensive first):
  // sets are dealt to the workgroups in turn instead of one contiguous range per XCD
  const int set_end = sets_per_xcd ? min(n_sets, (xcd + 1) * sets_per_xcd) : n_sets;

  // The next group of (up to) four taps out of `rest`: their numbers packed one per byte (K for
  // an unused slot), and the OR of their bits.
  struct Group {
    unsigned packed, bits;
  };
  auto pop_group = [&](unsigned &rest) {
    Group G;
    G.packed = 0;
    G.bits = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const unsigned k = min((unsigned)(__ffs((int)rest) - 1), (unsigned)K);  // no bit left: K
      G.bits |= rest & (0u - rest);
      rest &= rest - 1u;
      G.packed |= k << (8 * j);
    }
    return G;
  };
  // indices of a group for the four granules of the set starting at position t0
  auto load_idx = [&](const Group &G, unsigned t0, int *idx) {
    const unsigned tap = (G.packed >> shift8) & 0xFFu;
    const unsigned voff = tap * tap_stride + (t0 + (unsigned)r16) * 4u;  // tap K: past the end, reads 0
#pragma unroll
    for (int q = 0; q < 4; q++) idx[q] = __builtin_amdgcn_raw_buffer_load_b32(nbr_rsrc, voff + q * 64, 0, 0);
  };
  auto gather = [&](const Group &G, const int *idx, Row *a) {
    const unsigned tap = (G.packed >> shift8) & 0xFFu;
    const bool unused = tap == (unsigned)K;
    // an unused slot of a group reads past the end (zeros); a group without any tap is never
    // multiplied: its lanes all read row 0, which costs one access instead of 64
    const unsigned nowhere = G.bits ? 0x80000000u : 0u;
#pragma unroll
    for (int q = 0; q < 4; q++) {
      // j * ROW_BYTES as an unsigned offset: -1 (no neighbour) lands near 2^32, past any buffer this kernel is launched on
      const unsigned voff = min((unsigned)__mul24(idx[q], ROW_BYTES), 0x80000000u);
      a[q] = load_row<NIN>(in_rsrc, unused ? nowhere : voff);
    }
  };

  for (int sw = 0; sw < sets_per_wave; sw++) {
    const int set = sets_per_xcd ? xcd * sets_per_xcd + (blk * sets_per_wave + sw) * 4 + wave
                                 : ((int)blockIdx.x * sets_per_wave + sw) * 4 + wave;  // wave-uniform
    if (set >= set_end) break;
    unsigned gm[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int64_t gi = (int64_t)set * 4 + q;
      gm[q] = gi < n_granules ? gmask[gi] : 0u;
    }
    unsigned rest = gm[0] | gm[1] | gm[2] | gm[3];
    const int n_groups = (__builtin_popcount(rest) + 3) >> 2;  // 0: a set without rules takes one empty group
    const unsigned t0 = (unsigned)set * 64u;
    v4f acc[4][NCB];
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
      for (int cb = 0; cb < NCB; cb++) acc[q][cb] = (v4f){0.f, 0.f, 0.f, 0.f};

    int i0[4], i1[4];
    Row a0[4], a1[4];
    auto mfmas = [&](const Group &G, const Row *a) {
      const unsigned tap = (G.packed >> shift8) & 0xFFu;
      const float *wsrc = wl + tap * (unsigned)WS + r16;
      float b[NIN][NCB];
#pragma unroll
      for (int c = 0; c < NIN; c++)
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) b[c][cb] = wsrc[(c * NCB + cb) * 16];
#pragma unroll
      for (int q = 0; q < 4; q++) {
        if ((gm[q] & G.bits) == 0u) continue;  // uniform: no row of this granule has one of the taps
#pragma unroll
        for (int c = 0; c < NIN; c++)
#pragma unroll
          for (int cb = 0; cb < NCB; cb++)
            acc[q][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(plane_of<NIN>(a[q], c), b[c][cb], acc[q][cb], 0, 0, 0);
      }
    };
    // Software pipeline over the set's groups, two deep: while a group's MFMAs run, the next
    // group's rows and the indices of the one after are in flight.  All loads of the loop are
    // unconditional, so that the compiler can count them (a wait is a count of loads that may
    // still be outstanding); groups past the set's last have no taps, their index loads read
    // nothing and their gathers all read row 0 (one access).  A trip issues its index loads before
    // its gathers: waiting for indices (the counter is in order) then does not wait for rows.
    // Two groups per trip: the two register sets swap roles without copies.
    Group G0 = pop_group(rest);
    load_idx(G0, t0, i0);
    Group G1 = pop_group(rest);
    load_idx(G1, t0, i1);
    gather(G0, i0, a0);
    for (int gi = 0;;) {
      Group G2 = pop_group(rest);
      load_idx(G2, t0, i0);
      gather(G1, i1, a1);
      mfmas(G0, a0);
      if (++gi >= n_groups) break;
      G0 = pop_group(rest);
      load_idx(G0, t0, i1);
      gather(G2, i0, a0);
      mfmas(G1, a1);
      if (++gi >= n_groups) break;
      const Group T = G0;
      G0 = G2;
      G1 = T;
    }
    // acc[q][cb][r]: position t0 + 16 q + 4 g + r, column 16 cb + r16.  A store instruction
    // writes 64 consecutive bytes of each of four rows.  (Measured no faster: the transposed
    // product, whose lanes hold four columns of a row of their own, and 16-byte stores after a
    // transposition inside quads of lanes.)
    unsigned roff[4][4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const unsigned p0 = t0 + 16u * q + 4u * g;
      int rows[4];
      if (rowmap) {
        const int4 rm = *reinterpret_cast<const int4 *>(rowmap + p0);  // p0 + 3 < npad
        rows[0] = rm.x, rows[1] = rm.y, rows[2] = rm.z, rows[3] = rm.w;
      } else {
#pragma unroll
        for (int r = 0; r < 4; r++) rows[r] = (int)(p0 + r);
      }
#pragma unroll
      for (int r = 0; r < 4; r++)
        roff[q][r] = (int64_t)(p0 + r) < n ? __umul24((unsigned)rows[r], out_row_bytes) : 0x80000000u;
    }
    // the two halves of a row are stored back to back (they merge on their way to memory);
    // only the last column block can have lanes whose column does not exist: they store nothing
    const bool last_ok = 16 * (NCB - 1) + r16 < n_out;
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
      for (int r = 0; r < 4; r++)
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) {
          if (cb == NCB - 1 && !last_ok) continue;
          float v = acc[q][cb][r] + bv[cb];
          if (post) v = epi_act(v, es[cb], eh[cb], leak);
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v), out_rsrc, roff[q][r] + col_off[cb], 0, 0);
        }
  }
}

static bool first_serves(const Table &t, int64_t in_rows, int n_in, int n_out) {
  if (t.K > 32 || n_in > 4 || n_out > 32 || t.gmask.p == nullptr || t.n == 0) return false;
  // what the 32-bit offsets of the buffer loads and stores reach: signed 24-bit row numbers,
  // everything below 2 GiB
  const int64_t in_bytes = in_rows * n_in * 4, nbr_bytes = (int64_t)t.K * t.npad * 4, out_bytes = t.n * n_out * 4;
  const int64_t lim = ((int64_t)1 << 31) - 4096;
  return in_rows > 0 && in_rows < (1 << 23) && t.n < (1 << 24) && in_bytes < lim && nbr_bytes < lim && out_bytes < lim;
}

bool conv_first_serves(const Table &t, int64_t in_rows, int n_in, int n_out) { return first_serves(t, in_rows, n_in, n_out); }

template <int NIN, int NCB>
static void launch_first(const Table &t, const float *in, int64_t in_rows, float *out, const float *w, const float *bias,
                         CoefJob bn, float leak, int n_out, hipStream_t s) {
  const int64_t in_bytes = in_rows * NIN * 4, nbr_bytes = (int64_t)t.K * t.npad * 4, out_bytes = t.n * n_out * 4;
  const int n_sets = (int)ceil_div(t.n, 64);
  const int sets_per_xcd = t.spread ? 0 : (int)ceil_div(n_sets, 8);
  // one set per wavefront: measured best (the hardware's workgroup dispatch evens out the sets'
  // different tap counts)
  const int spw = 1;
  const int blocks = sets_per_xcd ? 8 * (int)ceil_div(sets_per_xcd, 4 * spw) : (int)ceil_div(n_sets, 4 * spw);
  k_conv_first<NIN, NCB><<<dim3(blocks), 256, (size_t)(t.K + 1) * first_tap_floats(NIN, NCB) * sizeof(float), s>>>(
      t.nbr.p, t.rowmap_ptr(), t.gmask.p, t.K, t.n, t.npad, in, out, w, bias, bn, leak, n_out, n_sets, sets_per_xcd, spw,
      (unsigned)in_bytes, (unsigned)nbr_bytes, (unsigned)out_bytes);
  LAUNCH_CHECK();
}

// bn.n == 0: no batch norm behind the convolution.
void conv_first_forward(const Table &t, const float *in, int64_t in_rows, float *out, const float *w, const float *bias,
                        CoefJob bn, float leak, int n_in, int n_out, hipStream_t s) {
  if (!first_serves(t, in_rows, n_in, n_out)) throw Error("internal: first-layer kernel asked for a shape it does not serve");
#define SCN_FIRST(NIN)                                                                     \
  do {                                                                                     \
    if (n_out <= 16) launch_first<NIN, 1>(t, in, in_rows, out, w, bias, bn, leak, n_out, s); \
    else launch_first<NIN, 2>(t, in, in_rows, out, w, bias, bn, leak, n_out, s);           \
  } while (0)
  if (n_in == 1) SCN_FIRST(1);
  else if (n_in == 2) SCN_FIRST(2);
  else if (n_in == 3) SCN_FIRST(3);
  else SCN_FIRST(4);
#undef SCN_FIRST
}

}  // namespace scn
