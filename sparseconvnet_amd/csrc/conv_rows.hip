// The row-owner MFMA convolution kernel (mid-width layers) and its dispatch; see conv.hip for the family.
#include "conv_common.h"

namespace scn {

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
    int n_split, int split_tiles, float *__restrict__ partial, const float *__restrict__ pre_sc,
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

  SCN_PHASE(0);  // start
  // The taps of the first split_tiles tiles are dealt over n_split workgroups each (`split`: which of
  // them this is, -1: the tile is this workgroup's alone).  Levels of fewer than 256 tiles split
  // all their tiles, to fill the chip.
  int tile, split;
  if (tiles_per_xcd) {
    tile = (blockIdx.x & 7) * tiles_per_xcd + (blockIdx.x >> 3);
    split = n_split > 1 ? (int)blockIdx.y : -1;
  } else if ((int)blockIdx.x < split_tiles * n_split) {
    tile = blockIdx.x % split_tiles;
    split = blockIdx.x / split_tiles;
  } else {
    tile = split_tiles + ((int)blockIdx.x - split_tiles * n_split);
    split = -1;
  }
  const int ways = split < 0 ? 1 : n_split;
  if (tile >= n_tiles) return;
  const int64_t tbase = (int64_t)tile * TM;

  const int ntaps = tile_setup<NT, G>(nbr, K, n, npad, tbase, ways, split, jtab, gmask, taplist, ntaps_p);
  const int total = ntaps * n_slab;
  SCN_PHASE(1);  // tile set up
  SCN_PHASE_VALUE(7, total);
  // Filters of up to 64 taps: the tap list and the taps of this wavefront's granules as bit masks in
  // scalar registers, so that the tap of an iteration and whether a granule has it are scalar
  // arithmetic instead of LDS reads on the path from the barrier to the first MFMA.
  const bool small_k = K <= 64;
  unsigned long long tmask = 0ull, mym[RG];
#pragma unroll
  for (int q = 0; q < RG; q++) mym[q] = 0ull;
  if (small_k) {
    const unsigned gmv = lane < K ? gmask[lane] : 0u;
    tmask = __ballot(gmv != 0u && (ways == 1 || lane % ways == split));
#pragma unroll
    for (int q = 0; q < RG; q++) mym[q] = __ballot((gmv >> (wave * RG + q)) & 1u) & tmask;
  }
  v4f acc[RG][NCB];
#pragma unroll
  for (int q = 0; q < RG; q++)
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) acc[q][cb] = (v4f){0.f, 0.f, 0.f, 0.f};

  // Loads in flight: the weight slab one iteration ahead (it comes from L2), the gathered rows AD
  // iterations ahead, in a ring of register sets (the loop below is unrolled AD times so that the
  // set is a constant).  On a level whose rows an XCD does not keep in its L2 a gather takes longer
  // than the MFMAs of one iteration (0.7 us at 96 output planes); measured 5 % at 60 k sites.
  // Two granules per wavefront (the 128-row tiles of million-site levels, whose gathers mostly hit
  // L2): one iteration of look-ahead, as the ring's registers would cost a wavefront per SIMD.
  constexpr int AD = RG == 1 ? 3 : 1;
  v4f wreg[WPT];
  v4f a_ring[AD][RG][SS];
  unsigned gm_ring[AD] = {}, ok_ring[AD] = {};
  int sl_ring[AD] = {};
  v4f a_cur[RG][WS];  // bf16: the eight values of a pair of steps
  v4f psc[SS], psh[SS];
  unsigned gm_cur = 0;

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
  // Two cursors over the iterations (slab outer, tap inner: see k_conv_mfma), one for the weights
  // and one for the rows.  Both stay on the last iteration once they reach it: the loads are
  // issued unconditionally (a few re-read the last iteration's operands at the end of a tile), so
  // the number of loads in flight at every wait is a constant the compiler can count on.
  int w_ti = 0, w_sl = 0, w_left = total;
  int a_ti = 0, a_sl = 0, a_left = total;
  unsigned long long w_rest = tmask, a_rest = tmask;  // small_k: taps of the current slab still to come
  // The tap at a cursor, and the cursor's step to the next iteration (it stays on the last one).
  auto tap_at = [&](int ti, unsigned long long rest) {
    return small_k ? (int)__builtin_ctzll(rest | (1ull << 63)) : __builtin_amdgcn_readfirstlane(taplist[ti]);
  };
  auto advance = [&](int &ti, int &sl, int &left, unsigned long long &rest) {
    if (--left > 0) {
      rest &= rest - 1ull;
      if (++ti == ntaps) {  // slab outer, tap inner (see k_conv_mfma)
        ti = 0;
        sl++;
        rest = tmask;
      }
    }
  };
  // Neighbour rows of the iteration at the rows' cursor, read from LDS one call ahead of their use.
  int j_pre[RG];
  auto prefetch_j = [&]() {
    const int k = tap_at(a_ti, a_rest);
#pragma unroll
    for (int q = 0; q < RG; q++) j_pre[q] = jtab[((wave * RG + q) * K + k) * 16 + ld_row];
  };
  // (Past the end the loads ask for an offset outside their buffer, which the hardware answers with
  // zeros without touching memory: a strided table's tiles have one or two iterations, and re-reading
  // operands three times over would double their traffic.)
  const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(wp), 0, (int)min((int64_t)K * n_slab * SLAB_STRIDE_F4 * 16, (int64_t)0x7FFFFFFF), 0x00020000);
  auto issue_w = [&]() {
    const int sl = w_sl;
    const bool live = w_left > 0;
    // LDS values every lane reads alike: tell the compiler, so that what follows from them
    // (weight address, branches on the granule mask) is scalar work
    const int k = tap_at(w_ti, w_rest);
    advance(w_ti, w_sl, w_left, w_rest);
    if (PRE) {
#pragma unroll
      for (int s = 0; s < SS; s++) {
        psc[s] = *reinterpret_cast<const v4f *>(pre_sc + (sl * SS + s) * 16 + 4 * ld_g);
        psh[s] = *reinterpret_cast<const v4f *>(pre_sh + (sl * SS + s) * 16 + 4 * ld_g);
      }
    }
    // The slab's byte offset goes in the scalar operand, the lane's part in the vector operand; only
    // the vector operand is checked against the buffer's size, so that is where "past the end" goes.
    const unsigned sbase = (unsigned)(k * n_slab + sl) * (unsigned)(SLAB_STRIDE_F4 * 16);
#pragma unroll
    for (int i = 0; i < WPT; i++) {
      const int e = threadIdx.x + i * NT;
      const unsigned voff = live ? (unsigned)(e < SLAB_F4 ? e : 0) * 16u : 0x80000000u;
      wreg[i] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, voff, sbase, 0));
    }
  };
  auto issue_a = [&](auto stage_c) {
    constexpr int S = decltype(stage_c)::value;
    const int sl = a_sl;
    const bool live = a_left > 0;
    const int k = tap_at(a_ti, a_rest);
    advance(a_ti, a_sl, a_left, a_rest);
    // bit q: granule q of this wavefront has the tap
    if (small_k) {
      gm_ring[S] = 0u;
#pragma unroll
      for (int q = 0; q < RG; q++) gm_ring[S] |= (unsigned)((mym[q] >> k) & 1ull) << q;
    } else {
      gm_ring[S] = (__builtin_amdgcn_readfirstlane(gmask[k]) >> (wave * RG)) & ((1u << RG) - 1u);
    }
    sl_ring[S] = sl;
    ok_ring[S] = 0;
    int jq[RG];
#pragma unroll
    for (int q = 0; q < RG; q++) jq[q] = j_pre[q];
    prefetch_j();  // for the next call
#pragma unroll
    for (int q = 0; q < RG; q++) {
      const int j = jq[q];
      if constexpr (BUF) {
        // Buffer loads return zeros past the end of the buffer: an absent row becomes an
        // offset of 2 GiB (the launcher only takes this path for smaller inputs, whole slabs
        // and fewer than 2^24 rows), so no select is needed afterwards and the address is
        // one 24-bit multiply-add.
        const unsigned voff = (j >= 0 && live) ? __umul24((unsigned)j, row_bytes) + lane_off : 0x80000000u;
        if (PRE && j >= 0) ok_ring[S] |= 1u << q;  // zero must stay zero through the pre-activation
#pragma unroll
        for (int s = 0; s < SS; s++)
          a_ring[S][q][s] = __builtin_bit_cast(
              v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, (sl * SS + s) * 64, 0));
        continue;
      }
      if (j >= 0) ok_ring[S] |= 1u << q;
      const float *src = in + (int64_t)(j < 0 ? 0 : j) * n_in;
#pragma unroll
      for (int s = 0; s < SS; s++) {
        const int c0 = (sl * SS + s) * 16 + 4 * g;
        if (VEC4) {
          const int cc = c0 < n_in ? c0 : n_in - 4;
          a_ring[S][q][s] = *reinterpret_cast<const v4f *>(src + cc);
        } else {
          a_ring[S][q][s].x = src[min(c0 + 0, n_in - 1)];
          a_ring[S][q][s].y = src[min(c0 + 1, n_in - 1)];
          a_ring[S][q][s].z = src[min(c0 + 2, n_in - 1)];
          a_ring[S][q][s].w = src[min(c0 + 3, n_in - 1)];
        }
      }
    }
  };

  // One iteration: the weights of `it` go to LDS, its rows (ring set S) to the operand registers,
  // then the loads of the iterations ahead are issued and the MFMAs run.
  auto iterate = [&](int it, auto stage_c) {
    constexpr int S = decltype(stage_c)::value;
    v4f *wb = wbuf + (it & 1) * LDS_SLAB_F4;
#pragma unroll
    for (int i = 0; i < WPT; i++) wb[threadIdx.x + i * NT] = wreg[i];
#pragma unroll
    for (int q = 0; q < RG; q++) {
      const bool ok = (ok_ring[S] >> q) & 1u;
      if constexpr (BF16) {
#pragma unroll
        for (int s = 0; s < SS; s += 2) {
          v4f v0 = a_ring[S][q][s], v1 = a_ring[S][q][s + 1];
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
          a_cur[q][s] = to_operand_lanes(a_ring[S][q][s]);
          continue;
        }
        if constexpr (BUF && PRE && !BF16) {
          const v4f v = pre_act<PRE>(a_ring[S][q][s], psc[s], psh[s], pre_leak);
          a_cur[q][s] = to_operand_lanes(ok ? v : (v4f){0.f, 0.f, 0.f, 0.f});
          continue;
        }
        if constexpr (!BUF) {
          const int c0 = (sl_ring[S] * SS + s) * 16 + 4 * g;
          v4f v = pre_act<PRE>(a_ring[S][q][s], psc[s], psh[s], pre_leak);
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
    gm_cur = gm_ring[S];
    __syncthreads();  // slab of `it` visible; every wavefront is done with the other buffer
    issue_w();
    issue_a(stage_c);
    if (gm_cur == 0u) return;  // none of my granules has the tap
#pragma unroll
    for (int s = 0; s < WS; s++) {
      v4f b[NCB];
#pragma unroll
      for (int cb = 0; cb < NCB; cb++) b[cb] = wb[(s * NCB + cb) * 64 + lane];
#pragma unroll
      for (int q = 0; q < RG; q++) {
        if (!((gm_cur >> q) & 1u)) continue;  // uniform over the wavefront
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
  };

  static_assert(AD == 1 || AD == 3, "the loop is unrolled for a ring of one or three");
  if (total > 0) {
    prefetch_j();
    issue_a(std::integral_constant<int, 0>{});
    if constexpr (AD == 3) {
      issue_a(std::integral_constant<int, 1>{});
      issue_a(std::integral_constant<int, 2>{});
    }
    issue_w();
  }
  SCN_PHASE(2);  // first loads issued
  for (int it = 0; it < total; it += AD) {
    iterate(it, std::integral_constant<int, 0>{});
    if (it == 0) SCN_PHASE(3);  // first iteration done
    if constexpr (AD == 3) {
      if (it + 1 < total) iterate(it + 1, std::integral_constant<int, 1>{});
      if (it + 2 < total) iterate(it + 2, std::integral_constant<int, 2>{});
    }
  }
  SCN_PHASE(4);  // tap loop done
  if (split >= 0) {  // partial tiles: [n_split][split_tiles * TM][NCB * 16]
    float *pt = partial + ((int64_t)split * split_tiles * TM + tbase) * (NCB * 16);
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
        if (epi.out2 && col < n_out) epi_second(epi, row, col, v);
        if (post) v = epi_act(v, es[cb], eh[cb], epi.leak);
        if (col < n_out) o[col] = v;
      }
    }
  }
  SCN_PHASE(5);  // rows stored
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
    launch_pack_weights(w, dst, t.K, n_in, n_out, n_slab, SS, NCB, SLAB_STRIDE, take_jobs(m), BF16, s);
  });
  auto kern = k_conv_rows<NCB, RG, SS, VEC4, NW, PRE, BUF, BF16>;
  static bool attr_set = false;
  if (!attr_set) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  160 * 1024));
    attr_set = true;
  }
  const int n_tiles = (int)ceil_div(t.n, G * 16);
  const int tiles_per_xcd = t.spread ? 0 : (int)ceil_div(n_tiles, 8);  // 0: tile = workgroup index
  // Few tiles: deal the taps of every tile over several workgroups (about two per CU in all).
  // (Splitting only the most expensive tiles of a larger level, whose 27-tap tiles run three times
  // the iterations of its 9-tap ones, was measured slower at 61 k sites, 179 -> 192 us: the extra
  // workgroups no longer all fit on the chip at once.  The kernel keeps the means: split_tiles.)
  int n_split = 1, split_tiles = 0;
  if (n_tiles < 256) {
    n_split = (int)std::min<int64_t>(t.K, ceil_div(512, n_tiles));
    split_tiles = n_tiles;
  }
  const int64_t split_stride = (int64_t)split_tiles * G * 16 * NCB * 16;
  float *partial = scratch_partial(m, n_split, split_stride);
  if (n_split <= 1) n_split = 1, split_tiles = 0;
  note_kernel(m, BF16 ? "rows-bf16" : "rows", {{"ncb", NCB}, {"rg", RG}, {"ss", SS}, {"nw", NW}, {"pre", PRE}, {"split", n_split},
                                                {"split_tiles", split_tiles}});
  const dim3 grid = tiles_per_xcd ? dim3((unsigned)(tiles_per_xcd * 8), n_split)
                                  : dim3((unsigned)(split_tiles * n_split + (n_tiles - split_tiles)));
  kern<<<grid, NT, lds_bytes, s>>>(
      t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, in, out, wpack, epi, n_in, n_out, n_slab, tiles_per_xcd,
      n_tiles, n_split, split_tiles, partial, pre.sc, pre.sh, pre.leak, (unsigned)(m.cur_in_rows * n_in * 4));
  LAUNCH_CHECK();
  if (n_split > 1)
    launch_conv_reduce(partial, n_split, split_stride, NCB * 16, t.rowmap_ptr(), std::min<int64_t>(t.n, (int64_t)split_tiles * G * 16),
                       epi, out, n_out, s);
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
  // 128 output planes on a level of a few thousand to a few ten thousand sites: slabs of 64 input
  // channels halve the number of iterations (and barriers) of every tile; with one or two
  // workgroups per CU that is what counts (measured at 14 k sites: 128 -> 128 134 -> 110 us,
  // 256 -> 128 245 -> 192 us; no gain at 60 k and 250 k sites, where the larger slab costs a
  // resident workgroup per CU).
  if constexpr (VEC4) {
    if (!narrow && ncb > 6 && ncb <= 8 && t.n < 30000 && n_in % 64 == 0)
      return launch_rows<8, 1, 4, VEC4, 4, PRE>(m, t, in, out, w, epi, n_in, n_out, pre, s);
  }
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

bool conv_rows_dispatch(bool vec4, bool pre_fused, Metadata &m, const Table &t, const float *in, float *out,
                        const float *w, Epi epi, int n_in, int n_out, PreArgs pre, hipStream_t s) {
  if (pre_fused)
    return vec4 ? dispatch_rows<true, true>(m, t, in, out, w, epi, n_in, n_out, pre, s)
                : dispatch_rows<false, true>(m, t, in, out, w, epi, n_in, n_out, pre, s);
  return vec4 ? dispatch_rows<true, false>(m, t, in, out, w, epi, n_in, n_out, pre, s)
              : dispatch_rows<false, false>(m, t, in, out, w, epi, n_in, n_out, pre, s);
}

SCN_PHASE_EXPORT(scn_dbg_phases_rows)

}  // namespace scn
