// The resident-weights MFMA convolution kernel (narrow layers) and its dispatch; see conv.hip for the family.
#include "conv_common.h"

namespace scn {

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
    int sets_per_xcd, int accumulate, int *__restrict__ queue, unsigned in_bytes, unsigned nbr_bytes, int spread) {
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
  // spread (the table's positions are pattern-sorted as a whole, most expensive first): XCD x takes
  // the sets x, x + 8, x + 16, ... instead of a contiguous range, which would hand all the expensive
  // sets to the first XCD.  The stream below counts in the XCD's own numbering; set_of() gives the set.
  const int set_begin = xcd * sets_per_xcd;
  const int set_end = spread ? set_begin + max(0, (n_sets - xcd + 7) >> 3) : min(n_sets, set_begin + sets_per_xcd);
  auto set_of = [&](int i) { return min(spread ? (i - set_begin) * 8 + xcd : i, n_sets - 1); };
  const int first_round = blocks_per_xcd * WAVES;
  int *ctr = queue + xcd * 32;
  // Tables of few taps (strided and transposed convolutions: a set is one or a few items) take
  // eight sets per visit of the counter: one same-address atomic per set costs more than the set.
  const int chunk = K <= 8 ? 8 : 1;
  int chunk_next = 0, chunk_left = 0;
  auto take = [&]() {
    if (chunk_left == 0) {
      int v = 0;
      if (lane == 0) v = atomicAdd(ctr, chunk);
      chunk_next = set_begin + first_round + __builtin_amdgcn_readfirstlane(v);
      chunk_left = chunk;
    }
    chunk_left--;
    return chunk_next++;
  };
  // generator of the item stream (wave-uniform state)
  int g_set = set_begin + blk * WAVES + wave;
  bool g_has = g_set < set_end;
  unsigned g_rest = g_has ? set_mask(set_of(g_set)) : 0u;
  int g_next = take();           // the set after g_set
  unsigned g_mask_next = 0;      // its tap mask, read two items after g_next was requested
  int g_age = 0;
  struct Item {
    int k, set;
    bool last, valid;
  };
  auto gen = [&]() {
    if (++g_age == 2) g_mask_next = set_mask(set_of(g_next));
    Item it;
    it.valid = g_has;
    it.set = g_has ? set_of(g_set) : 0;
    it.k = g_has ? __ffs(g_rest) - 1 : 0;
    g_rest &= g_rest - 1;
    it.last = g_has && g_rest == 0u;
    if (it.last) {
      if (g_age < 2) g_mask_next = set_mask(set_of(g_next));  // a set of one or two taps
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
            float *o = out + row * (epi.out_stride ? epi.out_stride : n_out);
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) {
              const int col = 16 * cb + r16;
              if (col < n_out) {
                float v = acc[q][cb][r] + (accumulate ? o[col] : bv[cb]);
                if (epi.out2) epi_second(epi, row, col, v);
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
  note_kernel(m, BF16 ? "resident-bf16" : (C4 ? "resident-c4" : "resident"), {{"ncb", NCB}, {"rg", RG}, {"ss", SS}, {"waves", WAVES}});
  kern<<<dim3(blocks), WAVES * 64, lds_bytes, s>>>(t.nbr.p, t.rowmap_ptr(), t.gmask.p, t.K, t.n, t.npad, in, in_stride,
                                                   out, wpack, epi, n_in_part, n_out, n_sets, sets_per_xcd,
                                                   accumulate, scratch_queue(m, s), (unsigned)in_bytes, (unsigned)nbr_bytes, t.spread ? 1 : 0);
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
    launch_pack_weights_part(w, dst, t.K, w_in_stride_rows, n_in_part, n_out, SS, NCB, queue, take_jobs(m), bf16, s);
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
  if (in == m.cur_in_base && !epi.out_stride && !epi.out2 && conv_first_serves(t, m.cur_in_rows, n_in, n_out)) {
    // epi.sc / epi.sh point at arrays nobody fills on this path: the kernel folds the batch norm itself
    take_jobs(m);
    note_kernel(m, "first", {{"nin", n_in}});
    conv_first_forward(t, in, m.cur_in_rows, out, w, epi.bias, m.post_raw, epi.leak, n_in, n_out, s);
    return;
  }
  const int packed = t.K * NCB * 64;
  int *queue = scratch_queue(m, s);
  const float *wpack = packed_weights(m, {2, (int64_t)(uintptr_t)w, t.K, n_in, n_out, NCB}, packed, [&](float *dst) {
    launch_pack_weights_c4(w, dst, t.K, n_in, n_out, NCB, queue, take_jobs(m), s);
  });
  launch_resident_kernel<NCB, 4, 1, false, 8, true>(m, t, in, n_in, out, wpack, epi, n_in, n_out, 0,
                                                    (size_t)packed * sizeof(float), 3, s);
}

// Narrow layers: nOut <= 32, any nIn, K <= 32.  nIn is processed in parts of up to 32
// channels so that every part's weights fit in LDS; parts after the first accumulate.
// The resident kernel serves nOut <= 32 with up to 32 taps.  It takes the input channels in
// parts of 32 (every part after the first re-reads and re-writes the output) and has no fused
// batch norm, so from 64 input channels on the row-owner kernel is faster (measured).
bool resident_fits(const Metadata &m, const Table &t, int n_in, int n_out, bool with_bn) {
  if (!(t.K <= 32 && n_out <= 32 && t.gmask.p != nullptr)) return false;
  // the resident kernel computes in fp32 only; from two parts on the row-owner kernel's bf16
  // variant is faster (measured)
  if (m.bf16 && n_in >= 64 && n_in % 32 == 0) return false;
  // several parts re-read and re-write the output once per part: with few taps (strided and
  // transposed convolutions) that costs more than the convolution itself (and 64 planes as one part
  // of four slabs, whose weights still fit LDS, measured 115 us against the row-owner kernel's 94
  // for 64 -> 32 up to a million rows: a set of one tap is too small an item for this pipeline)
  if (n_in > 32 && t.K <= 8) return false;
  (void)with_bn;
  return n_in < 64;  // two parts and more: the row-owner kernel is 3 % (64 -> 32) to 10 % (96 -> 32) faster at 1 M sites
}

// No fused batch norm here: this kernel's time goes into the vector instructions around its
// small MFMA blocks, and normalising every gathered value (each row is gathered once per tap
// that reaches it) costs more than one extra pass over the rows.
bool try_resident(Metadata &m, const Table &t, const float *in, float *out, const float *w,
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
    b.out_stride = epi.out_stride;
    if (!acc) b.bias = epi.bias;
    if (c_lo + 32 >= n_in) {
      b.sc = epi.sc;
      b.sh = epi.sh;
      b.leak = epi.leak;
      b.out2 = epi.out2;
      b.out2_stride = epi.out2_stride;
      b.sc2 = epi.sc2;
      b.sh2 = epi.sh2;
      b.leak2 = epi.leak2;
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


}  // namespace scn
