// Transposed convolution of a filter = stride = 2 rulebook onto a wide, shallow level (2^dim taps,
// nIn <= 64, nOut <= 32: a U-Net's last up-sampling, CPU/Deconvolution.cpp:9-40 with
// Metadata/ConvolutionRules.h:19-31 read from the fine side).
//
// Every output position has exactly one rule: (tap, coarse row).  The general kernels treat that
// as a table of 2^dim columns of which one is filled: a tile reads all the columns, sets its tap
// list up behind two barriers, runs one or two iterations and stores, and nothing of that overlaps
// within a workgroup (measured at a million output sites: 91 us for 0.19 GB of operands).  Here
//   * the weights of all taps stay in LDS for the life of the workgroup (2^dim x nIn x nOut x 4
//     bytes: 64 KB at 8 x 64 x 32), read as B operands in the packed order of k_pack_weights;
//   * a wavefront owns a contiguous run of granules (16 positions of the tap-sorted table) and
//     takes each from its three index loads (tap, coarse row, output row: the table's columns
//     are never read) through the gather of 16 coarse rows and the MFMAs to the stores, with the
//     next two granules' rows and the rules of the next 64 positions in flight: no barrier after
//     the weights are in, nothing shared between wavefronts;
//   * a granule whose rows have different taps (the borders between the taps' runs) takes the
//     taps it has one after the other, with the rows of the other taps zeroed;
//   * every load and store of the loop is issued unconditionally (clamped addresses for what lies
//     past the end, buffer stores that drop rows and columns out of range): with a memory
//     instruction under a branch the compiler cannot count the operations in flight and waits
//     for all of them, which ends the look-ahead (measured: 79 us that way).
#include "conv_common.h"

namespace scn {

constexpr int FEW_THREADS = 512, FEW_WAVES = FEW_THREADS / 64;

template <int S, int NCB, bool IDENT>
__global__ __launch_bounds__(FEW_THREADS) void k_deconv_few(
    const unsigned char *__restrict__ ptap, const int *__restrict__ prow, const int *__restrict__ rowmap, int K,
    int64_t n, const float *__restrict__ in, float *__restrict__ out, const float *__restrict__ wp, Epi epi, int n_out,
    int64_t n_granules, int gran_per_wave, unsigned out_bytes, unsigned out2_bytes) {
  constexpr int SLAB_F4 = packed_slab_floats(S, NCB) / 4;
  constexpr int N_IN = S * 16;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  v4f *wl = reinterpret_cast<v4f *>(lds);  // [K][SLAB_F4]
  for (int e = threadIdx.x; e < K * SLAB_F4; e += FEW_THREADS) wl[e] = reinterpret_cast<const v4f *>(wp)[e];
  __syncthreads();  // the only barrier
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  float bv[NCB], es[NCB], eh[NCB], es2[NCB], eh2[NCB];
  unsigned col_off[NCB];  // byte offset of the lane's column in a row, or past any buffer
  const bool post = epi.sc != nullptr, second = epi.out2 != nullptr;
#pragma unroll
  for (int cb = 0; cb < NCB; cb++) {
    const int col = 16 * cb + r16;
    bv[cb] = (epi.bias != nullptr && col < n_out) ? epi.bias[col] : 0.0f;
    es[cb] = (post && col < n_out) ? epi.sc[col] : 1.0f;
    eh[cb] = (post && col < n_out) ? epi.sh[col] : 0.0f;
    es2[cb] = (second && col < n_out) ? epi.sc2[col] : 1.0f;
    eh2[cb] = (second && col < n_out) ? epi.sh2[col] : 0.0f;
    col_off[cb] = col < n_out ? 4u * (unsigned)col : 0x80000000u;
  }
  const unsigned out_row_bytes = 4u * (unsigned)(epi.out_stride ? epi.out_stride : n_out);
  const unsigned out2_row_bytes = 4u * (unsigned)epi.out2_stride;
  const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(out, 0, (int)out_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t out2_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(second ? epi.out2 : out, 0, (int)(second ? out2_bytes : 0u), 0x00020000);
  // Workgroups b, b + 8, ... run on one XCD: they take a contiguous range of the table, so that
  // the coarse rows the taps' runs of that range share are fetched into one L2.
  const int per_xcd = gridDim.x >> 3;  // the grid is a multiple of eight workgroups
  const int64_t widx = ((int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3)) * FEW_WAVES + wave;
  // a wavefront's run of the table in pieces of 64 positions (four granules): gran_per_wave is a multiple of four
  const int64_t n_quads = (n_granules + 3) >> 2;
  const int64_t q0 = widx * (gran_per_wave >> 2), q1 = min(n_quads, q0 + (int64_t)(gran_per_wave >> 2));
  if (q0 >= q1) return;

  // The rules of the 64 positions of piece Q, one per lane: tap (255: no rule), coarse row, output
  // row (-1 past the end).  Clamped addresses: the loads are unconditional.
  struct Idx {
    int tap, row, orow;
  };
  auto load_idx = [&](int64_t Q) {
    Idx x;
    const int64_t pos = Q * 64 + lane;
    const bool ok = Q < q1 && pos < n;
    const int64_t at = min(pos, n - 1);
    // IDENT (a 1x1 convolution's table): the rule of position t is (tap 0, row t), nothing to read
    const int tap = IDENT ? 0 : (int)ptap[at], row = IDENT ? (int)at : prow[at], orow = (!IDENT && rowmap) ? rowmap[at] : (int)at;
    x.tap = ok ? tap : 255;
    x.row = ok ? row : 0;
    x.orow = ok ? orow : -1;
    return x;
  };
  // The gather of granule q of a piece: lane (g, r16) reads channels 16 s + 4 g .. + 3 of the coarse
  // row of position 16 q + r16 (row 0 for a position without a rule; never multiplied).
  auto load_rows = [&](const Idx &x, int q, v4f (&a)[S]) {
    const int tap = __shfl(x.tap, 16 * q + r16, 64), row = __shfl(x.row, 16 * q + r16, 64);
    const float *src = in + (int64_t)(tap < K ? row : 0) * N_IN + 4 * g;
#pragma unroll
    for (int s = 0; s < S; s++) a[s] = *reinterpret_cast<const v4f *>(src + 16 * s);
  };
  // MFMAs and stores of granule q of a piece whose rows are in a.
  auto finish = [&](const Idx &x, int q, const v4f (&a)[S]) {
    const int my_tap = __shfl(x.tap, 16 * q + r16, 64);
    unsigned taps = 0;
    for (int k = 0; k < K; k++)
      if (__ballot(my_tap == k)) taps |= 1u << k;
    v4f acc[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) acc[cb] = (v4f){0.f, 0.f, 0.f, 0.f};
    while (taps) {
      const int k = __builtin_ctz(taps);
      taps &= taps - 1u;
      const v4f *wk = wl + k * SLAB_F4 + lane;
      const bool mine = my_tap == k;
#pragma unroll
      for (int s = 0; s < S; s++) {
        const v4f av = mine ? a[s] : (v4f){0.f, 0.f, 0.f, 0.f};
        v4f b[NCB];
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) b[cb] = wk[(s * NCB + cb) * 64];
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, b[cb].x, acc[cb], 0, 0, 0);
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, b[cb].y, acc[cb], 0, 0, 0);
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, b[cb].z, acc[cb], 0, 0, 0);
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, b[cb].w, acc[cb], 0, 0, 0);
      }
    }
    // acc[cb][i] = the value of position 16 q + 4 g + i of the piece, column 16 cb + r16
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int orow = __shfl(x.orow, 16 * q + 4 * g + i, 64);
      // a position past the end: an offset past the end of the buffer, the store is dropped
      const unsigned roff = orow < 0 ? 0x80000000u : (unsigned)orow * out_row_bytes;
      const unsigned roff2 = orow < 0 ? 0x80000000u : (unsigned)orow * out2_row_bytes;
#pragma unroll
      for (int cb = 0; cb < NCB; cb++) {
        float v = acc[cb][i] + bv[cb];
        // (a row and a column that are both out of range must not add up to offset 0)
        const bool drop = ((roff | col_off[cb]) & 0x80000000u) != 0u;
        if (second)  // uniform
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, epi_act(v, es2[cb], eh2[cb], epi.leak2)), out2_rsrc,
                                                drop ? 0x80000000u : roff2 + col_off[cb], 0, 0);
        if (post) v = epi_act(v, es[cb], eh[cb], epi.leak);
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v), out_rsrc, drop ? 0x80000000u : roff + col_off[cb], 0, 0);
      }
    }
  };

  // The rows of two granules are in flight while one is multiplied, in four register sets that
  // take turns by name (a set that is copied has to have arrived: no look-ahead survives a copy),
  // and the rules of the next piece while this one is worked on.
  Idx X = load_idx(q0), Y = load_idx(q0 + 1);
  v4f a0[S], a1[S], a2[S], a3[S];
  load_rows(X, 0, a0);
  load_rows(X, 1, a1);
  for (int64_t Q = q0; Q < q1; Q++) {
    load_rows(X, 2, a2);
    finish(X, 0, a0);
    load_rows(X, 3, a3);
    finish(X, 1, a1);
    load_rows(Y, 0, a0);  // past the end: row 0, never used
    finish(X, 2, a2);
    load_rows(Y, 1, a1);
    finish(X, 3, a3);
    X = Y;
    Y = load_idx(Q + 2);  // past the end: a clamped address, marked as no positions
  }
}

template <int S, int NCB, bool IDENT>
static bool launch_few(Metadata &m, const Table &t, const float *in, float *out, const float *w, Epi epi, int n_in,
                       int n_out, hipStream_t s) {
  constexpr int SLAB_STRIDE = packed_slab_floats(S, NCB);
  const size_t lds_bytes = (size_t)t.K * SLAB_STRIDE * sizeof(float);
  if (lds_bytes > 96 * 1024) return false;
  const int64_t packed = (int64_t)t.K * SLAB_STRIDE;
  float *wpack = packed_weights(m, {4, (int64_t)(uintptr_t)w, t.K, n_in, n_out, S, NCB, 0}, packed, [&](float *dst) {
    launch_pack_weights(w, dst, t.K, n_in, n_out, 1, S, NCB, SLAB_STRIDE, take_jobs(m), false, s);
  });
  auto kern = k_deconv_few<S, NCB, IDENT>;
  static bool attr_set = false;
  if (!attr_set) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    attr_set = true;
  }
  // the output rows are the table's positions in another order: t.n rows; buffer stores address 2 GiB
  const int64_t out_bytes = t.n * (int64_t)(epi.out_stride ? epi.out_stride : n_out) * 4;
  const int64_t out2_bytes = epi.out2 ? t.n * (int64_t)epi.out2_stride * 4 : 0;
  if (out_bytes >= ((int64_t)1 << 31) || out2_bytes >= ((int64_t)1 << 31)) return false;
  const int64_t n_granules = ceil_div(t.n, 16);
  // two workgroups per CU when there is enough to do: 4096 wavefronts, each a run of granules
  const int gran_per_wave = (int)round_up(std::max<int64_t>(1, ceil_div(n_granules, 4096)), 4);
  const int64_t waves = ceil_div(n_granules, gran_per_wave);
  const unsigned grid = (unsigned)round_up(ceil_div(waves, FEW_WAVES), 8);
  note_kernel(m, "few", {{"s", S}, {"ncb", NCB}, {"identity", IDENT}, {"granules_per_wave", gran_per_wave}});
  kern<<<dim3(grid), FEW_THREADS, lds_bytes, s>>>(t.few_tap.p, t.few_row.p, t.rowmap_ptr(), t.K, t.n, in, out, wpack, epi, n_out,
                                                  n_granules, gran_per_wave, (unsigned)out_bytes, (unsigned)out2_bytes);
  LAUNCH_CHECK();
  return true;
}

// Tables that carry their one rule per position (the fine side of a filter = stride = 2 rulebook,
// finish_by_in; the identity table of a 1x1 convolution, CPU/NetworkInNetwork.cpp:7-23) and shapes
// whose weights fit LDS; false: not for this kernel.
bool try_few(Metadata &m, const Table &t, const float *in, float *out, const float *w, Epi epi, int n_in, int n_out,
             hipStream_t s) {
  const bool ident = t.identity_few && t.identity_rows && t.K == 1;
  if ((!t.few_tap.p && !ident) || t.K > 8 || t.n <= 0 || m.bf16 || m.fixed_scratch) return false;
  if ((uintptr_t)in % 16 != 0) return false;
#define FEW_CASE(S, NCB)                                                                         \
  return ident ? launch_few<S, NCB, true>(m, t, in, out, w, epi, n_in, n_out, s)                 \
               : launch_few<S, NCB, false>(m, t, in, out, w, epi, n_in, n_out, s)
  if (n_in == 64 && n_out <= 32 && n_out > 16) FEW_CASE(4, 2);
  if (n_in == 64 && n_out <= 16) FEW_CASE(4, 1);
  if (n_in == 32 && n_out <= 32 && n_out > 16) FEW_CASE(2, 2);
  if (n_in == 32 && n_out <= 16) FEW_CASE(2, 1);
#undef FEW_CASE
  return false;
}

}  // namespace scn
