// Convolution forward, output-stationary: every output row accumulates, over the filter
// taps, the row its neighbour table names times that tap's weight slice, and is written
// exactly once (no atomics, no read-modify-write of the output, deterministic).
// One kernel family serves SubmanifoldConvolution, Convolution and Deconvolution
// (CPU/Convolution.cpp:45-79,117-150, CPU/Deconvolution.cpp:7-41); they differ only in
// the table they pass.
//
// MFMA kernel (groups == 1).  A workgroup owns WAVES*16 consecutive schedule positions;
// each wavefront owns a granule of 16 of them and keeps that granule's [16 x nOut]
// accumulators in registers for the whole filter.  Per tap the wavefront gathers its 16
// input rows straight from HBM/L2 into v_mfma_f32_16x16x4_f32 A-operand registers (16-byte
// loads; the reduction dimension is consumed in a lane-permuted order that the packed
// weights mirror), multiplies with the tap's weight slab that the workgroup has staged in
// LDS in B-operand order, and skips the tap altogether when none of its 16 rows has that
// neighbour.  Rows arrive in Z-order, so a granule's rows mostly share one neighbour
// pattern and the skipped taps carry almost all of the sparsity.
#include "metadata.h"

namespace scn {

typedef float v4f __attribute__((ext_vector_type(4)));

// ---- generic kernel: any channel counts, any groups -------------------------------------
__global__ void k_conv_generic(const int *nbr, const int *rowmap, int K, int64_t n, int64_t npad,
                               const float *in, float *out, const float *w, const float *bias, int n_in,
                               int n_out, int groups) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = n * n_out;
  if (i >= total) return;
  int64_t t = i / n_out;
  int oc = (int)(i - t * n_out);
  int ip = n_in / groups, op = n_out / groups;
  int g = oc / op, ocg = oc - g * op;
  float acc = bias ? bias[oc] : 0.0f;
  for (int k = 0; k < K; k++) {
    int j = nbr[(int64_t)k * npad + t];
    if (j < 0) continue;
    const float *x = in + (int64_t)j * n_in + g * ip;
    const float *wk = w + (((int64_t)k * groups + g) * ip) * op + ocg;
    float a = 0.0f;
    for (int c = 0; c < ip; c++) a += x[c] * wk[(int64_t)c * op];
    acc += a;
  }
  int64_t row = rowmap ? rowmap[t] : t;
  out[row * n_out + oc] = acc;
}

// ---- weight packing ---------------------------------------------------------------------
// wp[k][slab][s][cb][lane][jj] = W[k][channel (slab*SS+s)*16 + 4*(lane/16) + jj][16*cb + lane%16]
// (zero outside [nIn) x [nOut)): the order in which lane `lane` of a wavefront consumes B
// operands, so that staging a slab into LDS is a straight copy and each lane reads the four
// operands of one 16-channel step with a single 16-byte LDS load.
__global__ void k_pack_weights(const float *w, float *wp, int K, int n_in, int n_out, int n_slab, int SS,
                               int NCB) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = (int64_t)K * n_slab * SS * NCB * 256;
  if (i >= total) return;
  int jj = (int)(i & 3);
  int lane = (int)((i >> 2) & 63);
  int64_t r = i >> 8;
  int cb = (int)(r % NCB);
  r /= NCB;
  int s = (int)(r % SS);
  r /= SS;
  int sl = (int)(r % n_slab);
  int k = (int)(r / n_slab);
  int ch = (sl * SS + s) * 16 + 4 * (lane >> 4) + jj;
  int col = 16 * cb + (lane & 15);
  wp[i] = (ch < n_in && col < n_out) ? w[((int64_t)k * n_in + ch) * n_out + col] : 0.0f;
}

// ---- MFMA kernel ------------------------------------------------------------------------
template <int NCB, bool VEC4, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_conv_mfma(
    const int *__restrict__ nbr, const int *__restrict__ rowmap, int K, int64_t n, int64_t npad,
    const float *__restrict__ in, float *__restrict__ out, const float *__restrict__ wp,
    const float *__restrict__ bias, int n_in, int n_out, int n_slab, int SS, int tiles_per_xcd,
    int n_tiles) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int TM = WAVES * 16;
  int *tapflag = reinterpret_cast<int *>(lds + (size_t)SS * NCB * 256);  // [K]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, g = lane >> 4;

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of
  // tiles so that neighbouring tiles (which gather the same rows) share one L2.
  const int tile = (blockIdx.x & 7) * tiles_per_xcd + (blockIdx.x >> 3);
  if (tile >= n_tiles) return;  // whole workgroup leaves: no barrier is skipped
  const int64_t t0 = (int64_t)tile * TM + wave * 16;
  const int64_t t = t0 + r16;
  const bool live = t < n;

  for (int k = threadIdx.x; k < K; k += WAVES * 64) tapflag[k] = 0;
  __syncthreads();
  for (int k = 0; k < K; k++) {
    int j = live ? nbr[(int64_t)k * npad + t] : -1;
    if (__ballot(j >= 0) != 0ull && lane == 0) tapflag[k] = 1;
  }
  __syncthreads();

  v4f acc[NCB];
#pragma unroll
  for (int cb = 0; cb < NCB; cb++) acc[cb] = (v4f){0.f, 0.f, 0.f, 0.f};

  const int slab_f4 = SS * NCB * 64;  // float4 per slab
  for (int k = 0; k < K; k++) {
    if (!tapflag[k]) continue;  // uniform over the workgroup
    const int j = live ? nbr[(int64_t)k * npad + t] : -1;
    const bool wave_has = __ballot(j >= 0) != 0ull;
    const float *src = in + (int64_t)(j < 0 ? 0 : j) * n_in;
    for (int sl = 0; sl < n_slab; sl++) {
      __syncthreads();  // everyone is done with the previous slab
      const v4f *wsrc = reinterpret_cast<const v4f *>(wp) + ((int64_t)k * n_slab + sl) * slab_f4;
      for (int e = threadIdx.x; e < slab_f4; e += WAVES * 64) reinterpret_cast<v4f *>(lds)[e] = wsrc[e];
      __syncthreads();
      if (!wave_has) continue;  // uniform over the wavefront
      for (int s = 0; s < SS; s++) {
        const int c0 = (sl * SS + s) * 16 + 4 * g;
        v4f a = (v4f){0.f, 0.f, 0.f, 0.f};
        if (j >= 0) {
          if (VEC4) {
            if (c0 < n_in) a = *reinterpret_cast<const v4f *>(src + c0);
          } else {
            if (c0 + 0 < n_in) a.x = src[c0 + 0];
            if (c0 + 1 < n_in) a.y = src[c0 + 1];
            if (c0 + 2 < n_in) a.z = src[c0 + 2];
            if (c0 + 3 < n_in) a.w = src[c0 + 3];
          }
        }
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) {
          const v4f b = reinterpret_cast<const v4f *>(lds)[(s * NCB + cb) * 64 + lane];
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, acc[cb], 0, 0, 0);
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, acc[cb], 0, 0, 0);
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, acc[cb], 0, 0, 0);
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, acc[cb], 0, 0, 0);
        }
      }
    }
  }

  // acc[cb][r] = result for local row 4*g + r, column 16*cb + r16
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int64_t pos = t0 + 4 * g + r;
    if (pos >= n) continue;
    const int64_t row = rowmap ? rowmap[pos] : pos;
    float *o = out + row * n_out;
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) {
      const int col = 16 * cb + r16;
      if (col < n_out) o[col] = acc[cb][r] + (bias ? bias[col] : 0.0f);
    }
  }
}

template <int NCB, bool VEC4>
static void launch_mfma(Metadata &m, const Table &t, const int *rowmap, const float *in, float *out,
                        const float *w, const float *bias, int n_in, int n_out, hipStream_t s) {
  constexpr int WAVES = 4;
  const int cin16 = (int)ceil_div(n_in, 16);
  int SS = std::max(1, std::min(cin16, 32 / NCB));
  SS = std::min(SS, 8);
  const int n_slab = (int)ceil_div(cin16, SS);
  const int64_t packed = (int64_t)t.K * n_slab * SS * NCB * 256;
  m.wpack.reserve(packed);
  k_pack_weights<<<dim3((unsigned)ceil_div(packed, 256)), 256, 0, s>>>(w, m.wpack.p, t.K, n_in, n_out, n_slab,
                                                                      SS, NCB);
  LAUNCH_CHECK();
  const int n_tiles = (int)ceil_div(t.n, WAVES * 16);
  const int tiles_per_xcd = (int)ceil_div(n_tiles, 8);
  const size_t lds_bytes = (size_t)SS * NCB * 256 * sizeof(float) + (size_t)t.K * sizeof(int);
  k_conv_mfma<NCB, VEC4, WAVES><<<dim3((unsigned)(tiles_per_xcd * 8)), WAVES * 64, lds_bytes, s>>>(
      t.nbr.p, rowmap, t.K, t.n, t.npad, in, out, m.wpack.p, bias, n_in, n_out, n_slab, SS, tiles_per_xcd,
      n_tiles);
  LAUNCH_CHECK();
}

template <bool VEC4>
static bool dispatch_ncb(int ncb, Metadata &m, const Table &t, const int *rowmap, const float *in, float *out,
                         const float *w, const float *bias, int n_in, int n_out, hipStream_t s) {
#define SCN_CASE(N)                                                              \
  if (ncb <= N) {                                                                \
    launch_mfma<N, VEC4>(m, t, rowmap, in, out, w, bias, n_in, n_out, s);        \
    return true;                                                                 \
  }
  SCN_CASE(1) SCN_CASE(2) SCN_CASE(4) SCN_CASE(6) SCN_CASE(8) SCN_CASE(10) SCN_CASE(12) SCN_CASE(14) SCN_CASE(16)
#undef SCN_CASE
  return false;
}

void conv_forward(Metadata &m, const Table &t, const int *rowmap, const float *in, float *out, const float *w,
                  const float *bias, int n_in, int n_out, int groups, hipStream_t s) {
  if (groups < 1 || n_in < 1 || n_out < 1 || n_in % groups || n_out % groups)
    throw Error("channel counts must be positive multiples of groups");
  if (t.n == 0) return;
  if (groups == 1 && t.K <= 1024) {
    const int ncb = (int)ceil_div(n_out, 16);
    const bool vec4 = n_in % 4 == 0 && ((uintptr_t)in % 16 == 0);
    bool done = vec4 ? dispatch_ncb<true>(ncb, m, t, rowmap, in, out, w, bias, n_in, n_out, s)
                     : dispatch_ncb<false>(ncb, m, t, rowmap, in, out, w, bias, n_in, n_out, s);
    if (done) return;
  }
  int64_t total = t.n * n_out;
  k_conv_generic<<<dim3((unsigned)ceil_div(total, 256)), 256, 0, s>>>(t.nbr.p, rowmap, t.K, t.n, t.npad, in,
                                                                       out, w, bias, n_in, n_out, groups);
  LAUNCH_CHECK();
}

}  // namespace scn
