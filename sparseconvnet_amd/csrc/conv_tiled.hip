// The LDS-tiled MFMA convolution kernel (wide layers) and its dispatch; see conv.hip for the family.
#include "conv_common.h"

namespace scn {

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
  // tiles so that neighbouring tiles (which gather the same rows) share one L2.  Small levels
  // (tiles_per_xcd == 0, Table::spread) list their tiles most expensive first: workgroup i takes
  // tile i, so that the long tiles start first and on different CUs.
  SCN_PHASE(0);  // start
  const int tile = tiles_per_xcd ? (blockIdx.x & 7) * tiles_per_xcd + (blockIdx.x >> 3) : blockIdx.x;
  if (tile >= n_tiles) return;  // whole workgroup leaves: no barrier is skipped
  const int64_t tbase = (int64_t)tile * TM;

  const int ntaps = tile_setup<256, G>(nbr, K, n, npad, tbase, n_split, (int)blockIdx.y, jtab, gmask, taplist, ntaps_p);
  const int total = ntaps * n_slab;
  SCN_PHASE(1);  // tile set up
  SCN_PHASE_VALUE(7, total);
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
  SCN_PHASE(2);  // first loads issued
  for (int it = 0; it < total; it += 2) {
    iterate(it, std::integral_constant<int, 0>{});
    if (it == 0) SCN_PHASE(3);  // first iteration done
    if (it + 1 < total) iterate(it + 1, std::integral_constant<int, 1>{});
  }
  SCN_PHASE(4);  // tap loop done

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
    SCN_PHASE(5);  // partial tile stored
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
        if (epi.out2 && col < n_out) epi_second(epi, row, col, v);
        if (post) v = epi_act(v, es[c], eh[c], epi.leak);
        if (col < n_out) o[col] = v;
      }
    }
  }
}

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
    launch_pack_weights(w, dst, t.K, n_in, n_out, n_slab, SS, NCB, SLAB_STRIDE, take_jobs(m), BF16, s);
  });
  auto kern = k_conv_mfma<NCBW, WC, GW, SS, VEC4, PRE, BUF, BF16>;
  static bool attr_set = false;
  if (!attr_set) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  160 * 1024));
    attr_set = true;
  }
  const int n_tiles = (int)ceil_div(t.n, G * 16);
  const int tiles_per_xcd = t.spread ? 0 : (int)ceil_div(n_tiles, 8);  // 0: tile = workgroup index
  // Few tiles: deal the taps of every tile over several workgroups (about two per CU in all).
  int n_split = 1;
  // (three per CU of the 32-row tiles: 768, 1024 and 1536 workgroups measured alike, 512 slower)
  if (n_tiles < 256) n_split = (int)std::min<int64_t>(t.K, ceil_div(G == 2 ? 768 : 512, n_tiles));
  const int64_t split_stride = (int64_t)n_tiles * G * 16 * NCB * 16;
  float *partial = scratch_partial(m, n_split, split_stride);
  note_kernel(m, BF16 ? "tiled-bf16" : "tiled", {{"ncbw", NCBW}, {"wc", WC}, {"gw", GW}, {"ss", SS}, {"pre", PRE}, {"split", n_split}});
  kern<<<dim3((unsigned)(tiles_per_xcd ? tiles_per_xcd * 8 : n_tiles), n_split), 256, lds_bytes, s>>>(
      t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, in, out, wpack, epi, n_in, n_out, n_slab, tiles_per_xcd,
      n_tiles, n_split, partial, pre.sc, pre.sh, pre.leak, (unsigned)(m.cur_in_rows * n_in * 4));
  LAUNCH_CHECK();
  if (n_split > 1) launch_conv_reduce(partial, n_split, split_stride, NCB * 16, t.rowmap_ptr(), t.n, epi, out, n_out, s);
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
    // Below 8192 sites (fewer than 256 such tiles: the taps of a tile are dealt over several
    // workgroups) tiles of 32 rows with slabs of two steps: one workgroup's chain of MFMAs is what
    // such a launch lasts (152 rows x 224 planes: 81 workgroups of 10 us of MFMAs each on a chip of
    // 256 CUs), and halving the tile halves it.  Measured per convolution: 3.3 k sites x 160 planes
    // 68 -> 56 us, 320 -> 160 118 -> 89, 768 x 192 34.5 -> 32, 152 x 224 28.6 -> 22; 12.7 k x 160
    // (no tap split any more) 171 -> 191, hence the limit.
    if (t.n < 8192 && n_in % 32 == 0) {
      if (ncb <= 10) return launch_mfma<5, 2, 1, 2, VEC4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
      if (ncb <= 12) return launch_mfma<6, 2, 1, 2, VEC4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
      if (ncb <= 14) return launch_mfma<7, 2, 1, 2, VEC4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
      if (ncb <= 16) return launch_mfma<8, 2, 1, 2, VEC4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
    }
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


bool conv_tiled_dispatch(bool vec4, bool pre_fused, Metadata &m, const Table &t, const float *in, float *out,
                         const float *w, Epi epi, int n_in, int n_out, PreArgs pre, hipStream_t s) {
  const int ncb = (int)ceil_div(n_out, 16);
  if (pre_fused)
    return vec4 ? dispatch_ncb<true, true>(ncb, m, t, in, out, w, epi, n_in, n_out, pre, s)
                : dispatch_ncb<false, true>(ncb, m, t, in, out, w, epi, n_in, n_out, pre, s);
  return vec4 ? dispatch_ncb<true, false>(ncb, m, t, in, out, w, epi, n_in, n_out, pre, s)
              : dispatch_ncb<false, false>(ncb, m, t, in, out, w, epi, n_in, n_out, pre, s);
}

SCN_PHASE_EXPORT(scn_dbg_phases_tiled)

}  // namespace scn
