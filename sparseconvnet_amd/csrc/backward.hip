// Backward pass: gradients of the convolutions (with respect to input rows, weights and bias),
// of NetworkInNetwork, of batch normalisation in training mode (plus its training-mode forward),
// of the pooling layers, the input / output layers and sparse-to-dense.
//
// The reference computes these on the host per filter offset: gather rows, two GEMMs, scatter-add
// (CPU/Convolution.cpp:81-115,152-185, CPU/Deconvolution.cpp:43-77).  Here:
//   * the gradient of the input rows is itself an output-stationary convolution over a neighbour
//     table, with every tap's weight slice transposed: for a strided rulebook the table indexed
//     from the other side (the two tables of StridedRules list the same rules), for a
//     submanifold rulebook the same table with the taps mirrored (rule (k, i -> j) is rule
//     (K-1-k, j -> i)), so it runs through the forward kernels of conv.hip: no atomics,
//     deterministic;
//   * the gradient of the weights is, per tap, a [nIn x positions] x [positions x nOut] product
//     over the positions that have the tap: MFMA tiles over chunks of positions, partial sums per
//     chunk, then a reduction in fixed order (no float atomics, deterministic);
//   * column sums (bias gradients, batch-norm statistics) are two-stage reductions in fixed order.
#include "metadata.h"

namespace scn {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v3f __attribute__((ext_vector_type(3)));
static const int TB = 256;
static inline dim3 grid_for(int64_t n, int tb = TB) { return dim3((unsigned)std::max<int64_t>(1, ceil_div(n, tb))); }

// ---- transposed weights ------------------------------------------------------------------------
// wt[k'][g][o][c] = w[k][g][c][o], k' = K-1-k with mirror, else k.
__global__ void k_transpose_weights(const float *w, float *wt, int K, int groups, int ip, int op, int mirror) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t per = (int64_t)groups * ip * op;
  if (i >= K * per) return;
  const int k = (int)(i / per);
  int64_t r = i - k * per;
  const int g = (int)(r / ((int64_t)ip * op));
  r -= (int64_t)g * ip * op;
  const int o = (int)(r / ip), c = (int)(r - (int64_t)o * ip);
  const int ks = mirror ? K - 1 - k : k;
  wt[i] = w[(((int64_t)ks * groups + g) * ip + c) * op + o];
}

// ---- column sums -------------------------------------------------------------------------------
// partial[b][q][c] for row block b: q = 0: sum of a(row, c), q = 1: sum of b(row, c), where
//   MODE 0  a = x                                   (bias gradient; one quantity)
//   MODE 1  a = x, b = x * x                        (batch-norm statistics)
//   MODE 2  a = d * r, b = (x - mean[c]) * d * r    with r = out > 0 ? 1 : leak  (batch-norm backward)
// A workgroup of 256 threads covers CW columns by 256 * V / CW rows at a time; a thread owns V
// consecutive columns (V = 4: 16-byte loads, when the plane count and the row strides are
// multiples of four and the arrays 16-byte aligned) and has four rows in flight.
template <int MODE, int V>
__global__ __launch_bounds__(256) void k_colsum(const float *__restrict__ x, int64_t x_stride, const float *__restrict__ d,
                                                const float *__restrict__ out, int64_t o_stride,
                                                const float *__restrict__ mean, float leak, int64_t rows, int planes, int CW,
                                                int64_t rows_per_block, float *__restrict__ partial) {
  __shared__ float red[2][256 * V];
  const int TPR = CW / V;  // threads per row
  const int tx = threadIdx.x % TPR, ty = threadIdx.x / TPR, RW = 256 / TPR;
  const int c = blockIdx.y * CW + tx * V;
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block, r1 = min(rows, r0 + rows_per_block);
  float a[V], b[V];
#pragma unroll
  for (int v = 0; v < V; v++) a[v] = b[v] = 0.f;
  auto load = [&](const float *base, int64_t off, float (&dst)[V]) {
    if constexpr (V == 4) {
      const v4f t = *reinterpret_cast<const v4f *>(base + off);
      dst[0] = t.x, dst[1] = t.y, dst[2] = t.z, dst[3] = t.w;
    } else {
      dst[0] = base[off];
    }
  };
  if (c < planes) {
    float mu[V];
#pragma unroll
    for (int v = 0; v < V; v++) mu[v] = MODE == 2 ? mean[c + v] : 0.f;
    auto row = [&](int64_t r) {
      float xv[V], dv[V], ov[V];
      if (MODE != 2) {
        load(x, r * x_stride + c, xv);
#pragma unroll
        for (int v = 0; v < V; v++) {
          a[v] += xv[v];
          if (MODE == 1) b[v] += xv[v] * xv[v];
        }
      } else {
        load(d, r * o_stride + c, dv);
        load(out, r * o_stride + c, ov);
        load(x, r * x_stride + c, xv);
#pragma unroll
        for (int v = 0; v < V; v++) {
          const float g = dv[v] * (ov[v] > 0.f ? 1.f : leak);
          a[v] += g;
          b[v] += (xv[v] - mu[v]) * g;
        }
      }
    };
    int64_t r = r0 + ty;
    for (; r + 3 * RW < r1; r += 4 * RW) {  // four independent rows per trip
      row(r);
      row(r + RW);
      row(r + 2 * RW);
      row(r + 3 * RW);
    }
    for (; r < r1; r += RW) row(r);
  }
#pragma unroll
  for (int v = 0; v < V; v++) {
    red[0][threadIdx.x * V + v] = a[v];
    red[1][threadIdx.x * V + v] = b[v];
  }
  __syncthreads();
  // red[q][(ty * TPR + tx) * V + v] = column tx * V + v of row group ty: thread t < CW adds up column t
  if (threadIdx.x < CW && blockIdx.y * CW + threadIdx.x < planes) {
    float sa = 0.f, sb = 0.f;
    for (int q = 0; q < RW; q++) {
      sa += red[0][q * CW + threadIdx.x];
      sb += red[1][q * CW + threadIdx.x];
    }
    float *p = partial + (size_t)blockIdx.x * 2 * planes;
    p[blockIdx.y * CW + threadIdx.x] = sa;
    p[planes + blockIdx.y * CW + threadIdx.x] = sb;
  }
}
// Launches k_colsum<MODE, 4> when every operand allows 16-byte loads, else <MODE, 1>.
template <int MODE>
static void launch_colsum(dim3 grid, hipStream_t s, const float *x, int64_t x_stride, const float *d, const float *out,
                          int64_t o_stride, const float *mean, float leak, int64_t rows, int planes, int CW,
                          int64_t rows_per_block, float *partial) {
  auto ok = [](const float *p, int64_t stride) { return p == nullptr || ((uintptr_t)p % 16 == 0 && stride % 4 == 0); };
  if (planes % 4 == 0 && ok(x, x_stride) && ok(d, o_stride) && ok(out, o_stride))
    k_colsum<MODE, 4><<<grid, 256, 0, s>>>(x, x_stride, d, out, o_stride, mean, leak, rows, planes, CW, rows_per_block, partial);
  else
    k_colsum<MODE, 1><<<grid, 256, 0, s>>>(x, x_stride, d, out, o_stride, mean, leak, rows, planes, CW, rows_per_block, partial);
  LAUNCH_CHECK();
}
struct ColsumPlan {
  int CW, blocks;
  int64_t rows_per_block;
};
static ColsumPlan colsum_plan(int64_t rows, int planes) {
  ColsumPlan p;
  p.CW = planes <= 16 ? 16 : planes <= 32 ? 32 : 64;
  const int col_blocks = (int)ceil_div(planes, p.CW);
  // about four workgroups per CU in all, at least 256 rows each
  int64_t blocks = std::max<int64_t>(1, std::min<int64_t>(ceil_div(rows, 256), 1024 / col_blocks));
  p.rows_per_block = round_up(ceil_div(rows, blocks), 256 / p.CW);
  p.blocks = (int)ceil_div(rows, p.rows_per_block);
  return p;
}
// out[i] = sum over blocks b of partial[b * stride + i], i < count.  A workgroup of 1, 4 or 16
// wavefronts (blockDim.x / 64) takes 64 consecutive outputs: wavefront w adds up its contiguous
// share of the blocks in order, wavefront 0 then adds the shares in order (a fixed order: the
// result is the same on every run).  ACC is the accumulator type, OUT the type the sums are written in.
template <typename ACC, typename OUT>
__global__ __launch_bounds__(1024) void k_sum_blocks(const float *__restrict__ partial, int blocks, int64_t stride,
                                                     int64_t count, OUT *__restrict__ out) {
  __shared__ ACC part[16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t i = (int64_t)blockIdx.x * 64 + lane;
  const int waves = blockDim.x >> 6;
  const int per = (blocks + waves - 1) / waves;
  const int b0 = min(blocks, wave * per), b1 = min(blocks, b0 + per);
  ACC s = 0;
  if (i < count) {
#pragma unroll 4
    for (int b = b0; b < b1; b++) s += (ACC)partial[(size_t)b * stride + i];
  }
  part[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && i < count) {
    ACC tot = 0;
    for (int w = 0; w < waves; w++) tot += part[w][lane];
    out[i] = (OUT)tot;
  }
}
// Wavefronts per workgroup of k_sum_blocks: every wavefront gets at least four blocks to add.
static inline unsigned sum_threads(int64_t blocks) { return blocks >= 64 ? 1024 : blocks >= 16 ? 256 : 64; }
// The two column sums of a batch-normalisation pass, in double, for the 64 columns of workgroup
// blockIdx.x (1024 threads): partial[b][q][c] summed over the row blocks b in the fixed order of
// k_sum_blocks.  Every thread of wavefront 0 returns with the sums of column blockIdx.x * 64 + lane.
__device__ inline void pair_sums64(const float *__restrict__ partial, int blocks, int planes, double &s1, double &s2) {
  __shared__ double part[2][16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const int per = (blocks + 15) / 16;
  const int b0 = min(blocks, wave * per), b1 = min(blocks, b0 + per);
  double a = 0, b = 0;
  if (c < planes)
#pragma unroll 4
    for (int i = b0; i < b1; i++) {
      a += (double)partial[(size_t)i * 2 * planes + c];
      b += (double)partial[(size_t)i * 2 * planes + planes + c];
    }
  part[0][wave][lane] = a;
  part[1][wave][lane] = b;
  __syncthreads();
  s1 = s2 = 0;
  if (wave == 0) {
#pragma unroll
    for (int w = 0; w < 16; w++) s1 += part[0][w][lane], s2 += part[1][w][lane];
  }
}
static void column_sums(Metadata &m, const float *x, int64_t rows, int planes, float *out, hipStream_t s) {
  if (planes <= 0) return;
  if (rows <= 0) {
    fill32(out, 0, planes, s);
    return;
  }
  const ColsumPlan p = colsum_plan(rows, planes);
  m.partial.reserve((size_t)p.blocks * 2 * planes);
  launch_colsum<0>(dim3(p.blocks, (unsigned)ceil_div(planes, p.CW)), s, x, planes, nullptr, nullptr, 0, nullptr, 0.f,
                                                                                 rows, planes, p.CW, p.rows_per_block,
                                                                                 m.partial.p);
  k_sum_blocks<double, float><<<dim3((unsigned)ceil_div(planes, 64)), 1024, 0, s>>>(m.partial.p, p.blocks, (int64_t)2 * planes, planes, out);
  LAUNCH_CHECK();
}

// ---- weight gradient ---------------------------------------------------------------------------
// dW[k][c][o] = sum over positions t with nbr[k][t] >= 0 of a[nbr[k][t]][c] * b[row(t)][o].
// One workgroup (4 wavefronts): tap k, positions [chunk * chunk_len, ...), channel tile 64 x 64.
// Per step of 32 positions the gathered rows of a and the rows of b go through LDS as
// [position][channel]; wavefront (wr, wc) owns the 32 x 32 quadrant and feeds
// v_mfma_f32_16x16x4_f32 with the channel along the matrix rows / columns and four positions
// along the contraction.  Steps none of whose positions has the tap are skipped by the table's
// granule masks.  The next step's rows are fetched into registers while the current one runs.
constexpr int DW_T = 64, DW_PS = 32, DW_LD = DW_T + 16;
template <bool VEC4>
__global__ __launch_bounds__(256) void k_conv_dw(const int *__restrict__ nbr, const int *__restrict__ rowmap,
                                                 const unsigned *__restrict__ gmask, int K, int64_t n, int64_t npad,
                                                 const float *__restrict__ a, int n_a, const float *__restrict__ b,
                                                 int n_b, int64_t chunk_len, float *__restrict__ partial) {
  __shared__ __attribute__((aligned(16))) float la[DW_PS * DW_LD], lb[DW_PS * DW_LD];
  const int k = blockIdx.y;
  const int tiles_o = (n_b + DW_T - 1) / DW_T;
  const int ct = blockIdx.z / tiles_o, ot = blockIdx.z % tiles_o;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int wr = wave >> 1, wc = wave & 1;
  const int64_t p0 = (int64_t)blockIdx.x * chunk_len, p1 = min(n, p0 + chunk_len);
  // staging role of this thread: position lp of the step, channels [4 * lc, 4 * lc + 4) of each tile
  const int lp = threadIdx.x >> 4, lc = threadIdx.x & 15;  // two positions per thread: lp and lp + 16
  v4f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

  auto step_has_tap = [&](int64_t t0) {
    if (gmask == nullptr) return true;
    const int64_t g0 = t0 >> 4, gl = (n - 1) >> 4;
    return (((gmask[min(g0, gl)] | gmask[min(g0 + 1, gl)]) >> k) & 1u) != 0u;
  };
  auto load4 = [&](const float *base, int64_t row, int width, int c0) {
    v4f v = (v4f){0.f, 0.f, 0.f, 0.f};
    if (row < 0) return v;
    const float *src = base + row * width;
    if (VEC4) {
      if (c0 < width) v = *reinterpret_cast<const v4f *>(src + c0);
    } else {
      if (c0 + 0 < width) v.x = src[c0 + 0];
      if (c0 + 1 < width) v.y = src[c0 + 1];
      if (c0 + 2 < width) v.z = src[c0 + 2];
      if (c0 + 3 < width) v.w = src[c0 + 3];
    }
    return v;
  };
  v4f ra[2], rb[2];
  auto fetch = [&](int64_t t0) {
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int64_t t = t0 + lp + 16 * h;
      int64_t ja = -1, jb = -1;
      if (t < p1) {
        ja = nbr[(int64_t)k * npad + t];
        jb = ja >= 0 ? (rowmap ? rowmap[t] : t) : -1;
      }
      ra[h] = load4(a, ja, n_a, ct * DW_T + 4 * lc);
      rb[h] = load4(b, jb, n_b, ot * DW_T + 4 * lc);
    }
  };
  // first step of the chunk that has the tap
  int64_t t_cur = p0;
  while (t_cur < p1 && !step_has_tap(t_cur)) t_cur += DW_PS;
  if (t_cur < p1) fetch(t_cur);
  while (t_cur < p1) {
    __syncthreads();  // the previous step's MFMAs have read LDS
#pragma unroll
    for (int h = 0; h < 2; h++) {
      *reinterpret_cast<v4f *>(&la[(lp + 16 * h) * DW_LD + 4 * lc]) = ra[h];
      *reinterpret_cast<v4f *>(&lb[(lp + 16 * h) * DW_LD + 4 * lc]) = rb[h];
    }
    __syncthreads();
    int64_t t_nxt = t_cur + DW_PS;
    while (t_nxt < p1 && !step_has_tap(t_nxt)) t_nxt += DW_PS;
    if (t_nxt < p1) fetch(t_nxt);
#pragma unroll
    for (int kk = 0; kk < DW_PS / 4; kk++) {
      float av[2], bv[2];
#pragma unroll
      for (int i = 0; i < 2; i++) av[i] = la[(4 * kk + g) * DW_LD + (2 * wr + i) * 16 + r16];
#pragma unroll
      for (int j = 0; j < 2; j++) bv[j] = lb[(4 * kk + g) * DW_LD + (2 * wc + j) * 16 + r16];
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
    t_cur = t_nxt;
  }
  // acc[i][j][r] = dW[k][ct*64 + (2wr+i)*16 + 4g + r][ot*64 + (2wc+j)*16 + r16] of this chunk
  float *pk = partial + ((size_t)blockIdx.x * K + k) * (size_t)n_a * n_b;
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int c = ct * DW_T + (2 * wr + i) * 16 + 4 * g + r, o = ot * DW_T + (2 * wc + j) * 16 + r16;
        if (c < n_a && o < n_b) pk[(size_t)c * n_b + o] = acc[i][j][r];
      }
}
// The same sums for narrow layers (both channel counts <= 32), where the kernel above spends its
// time re-reading: one workgroup per tap reads the rows of b once per tap, 27 times in all.  Here
// a workgroup of eight wavefronts takes a share of the positions and a 32 x 32 channel tile for
// ALL taps: wavefront w keeps the accumulators of taps w, w + 8, w + 16, w + 24 (16 registers
// each) and walks its share 16 positions (one granule of the tap masks) at a time, skipping the
// taps the granule does not have.  Nothing goes through LDS: the MFMA contracts over four positions,
// lane (r, g) supplies position 4 g + kk of the granule and, of that position's row, the two
// channels 2 r and 2 r + 1 as one 8-byte load (16 lanes read 128 consecutive bytes); instruction
// i of a pair takes component i, so that it computes the gradient's rows 2 * (MFMA row) + i, and
// likewise for the columns.  The rows of b are loaded once per granule and serve all its taps.
constexpr int DT_NW = 8, DT_T = 32, DT_SLOTS = 4, DT_BLOCK = 8;  // DT_BLOCK granules of 16 positions per turn
template <bool VEC2>
__global__ __launch_bounds__(DT_NW * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_conv_dw_taps(const int *__restrict__ nbr, const int *__restrict__ rowmap,
                                                             const unsigned *__restrict__ gmask, int K, int64_t n,
                                                             int64_t npad, const float *__restrict__ a, int n_a,
                                                             unsigned a_bytes, const float *__restrict__ b, int n_b,
                                                             unsigned b_bytes, float *__restrict__ partial) {
  const int tiles_o = (n_b + DT_T - 1) / DT_T;
  const int ct = blockIdx.y / tiles_o, ot = blockIdx.y % tiles_o;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  v4f acc[DT_SLOTS][2][2];
#pragma unroll
  for (int sl = 0; sl < DT_SLOTS; sl++)
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int j = 0; j < 2; j++) acc[sl][i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  const int ca = ct * DT_T + 2 * r16, cb = ot * DT_T + 2 * r16;
  // rows of a come through a buffer resource: an offset of 2^31 or more reads zeros, which serves
  // absent rules (negative row) and channels beyond the last
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a), 0, (int)a_bytes, 0x00020000);
  const unsigned nowhere = 0x80000000u, a_row_bytes = (unsigned)n_a * 4u;
  const unsigned ca0 = ca < n_a ? (unsigned)ca * 4u : nowhere, ca1 = ca + 1 < n_a ? (unsigned)ca * 4u + 4u : nowhere;
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(b), 0, (int)b_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t nbr_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<int *>(nbr), 0, (int)((unsigned)K * (unsigned)npad * 4u), 0x00020000);
  const unsigned b_row_bytes = (unsigned)n_b * 4u;
  const unsigned cb0 = cb < n_b ? (unsigned)cb * 4u : nowhere, cb1 = cb + 1 < n_b ? (unsigned)cb * 4u + 4u : nowhere;
  // two channels of row j (negative: zeros); every row offset there is lies below 2^31
  auto pair_of = [&](const __amdgpu_buffer_rsrc_t &rsrc, int j, unsigned row_bytes, unsigned c0, unsigned c1) {
    const unsigned row = (unsigned)j * row_bytes;
    if (VEC2) return __builtin_bit_cast(v2f, __builtin_amdgcn_raw_buffer_load_b64(rsrc, j < 0 ? nowhere : row + c0, 0, 0));
    v2f v;
    v.x = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, j < 0 ? nowhere : row + c0, 0, 0));
    v.y = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, j < 0 ? nowhere : row + c1, 0, 0));
    return v;
  };
  unsigned own = 0u;  // the taps this wavefront accumulates
#pragma unroll
  for (int sl = 0; sl < DT_SLOTS; sl++)
    if (wave + sl * DT_NW < K) own |= 1u << (wave + sl * DT_NW);
  // Workgroup x takes the blocks of DT_BLOCK granules x, x + gridDim.x, ...: every workgroup sees
  // every part of the pattern-sorted table, so that they all carry about the same number of rules.
  const int n_granules = (int)((n + 15) >> 4), n32 = (int)n;  // the host checks that 4 K npad < 2^31
  for (int gb = blockIdx.x * DT_BLOCK; gb < n_granules; gb += gridDim.x * DT_BLOCK) {
    const int ge = min(n_granules, gb + DT_BLOCK);
    for (int gi = gb; gi < ge; gi++) {
      const unsigned present = gmask[gi] & own;
      if (present == 0u) continue;  // uniform over the wavefront
      const int t0 = gi << 4;
      // this lane's four positions of the granule: t0 + 4 g + kk; first the index quads of the
      // wavefront's taps, then all gathers, then the MFMAs: two memory latencies per granule
      // (fetching the next granule's quads meanwhile costs more registers than there are at
      // four wavefronts per SIMD, and measured slower with fewer)
      int4 j4[DT_SLOTS];
      const unsigned toff = (unsigned)(t0 + 4 * g) * 4u;
#pragma unroll
      for (int sl = 0; sl < DT_SLOTS; sl++) {
        const int k = wave + sl * DT_NW;
        // a tap the granule does not have: an offset past the table, which reads zeros; made -1 below
        j4[sl] = __builtin_bit_cast(int4, __builtin_amdgcn_raw_buffer_load_b128(
                                              nbr_rsrc, ((present >> k) & 1u) ? toff : nowhere, (unsigned)k * (unsigned)npad * 4u, 0));
      }
      v2f bv[4];
      if (rowmap) {
        const int4 r4 = *reinterpret_cast<const int4 *>(rowmap + t0 + 4 * g);
        const int r[4] = {r4.x, r4.y, r4.z, r4.w};
#pragma unroll
        for (int kk = 0; kk < 4; kk++) bv[kk] = pair_of(b_rsrc, t0 + 4 * g + kk < n32 ? r[kk] : -1, b_row_bytes, cb0, cb1);
      } else {
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
          const int t = t0 + 4 * g + kk;
          bv[kk] = pair_of(b_rsrc, t < n32 ? t : -1, b_row_bytes, cb0, cb1);
        }
      }
      v2f av[DT_SLOTS][4];
#pragma unroll
      for (int sl = 0; sl < DT_SLOTS; sl++) {
        const int k = wave + sl * DT_NW;
        const bool has = (present >> k) & 1u;
        const int j[4] = {j4[sl].x, j4[sl].y, j4[sl].z, j4[sl].w};
#pragma unroll
        for (int kk = 0; kk < 4; kk++) av[sl][kk] = pair_of(a_rsrc, has ? j[kk] : -1, a_row_bytes, ca0, ca1);
      }
#pragma unroll
      for (int sl = 0; sl < DT_SLOTS; sl++) {
        const int k = wave + sl * DT_NW;
        if (!((present >> k) & 1u)) continue;  // uniform over the wavefront
#pragma unroll
        for (int kk = 0; kk < 4; kk++)
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int jx = 0; jx < 2; jx++)
              acc[sl][i][jx] =
                  __builtin_amdgcn_mfma_f32_16x16x4f32(av[sl][kk][i], bv[kk][jx], acc[sl][i][jx], 0, 0, 0);
      }
    }
  }
  // acc[sl][i][jx][r] = dW[k][ct*32 + 2 (4 g + r) + i][ot*32 + 2 r16 + jx] of this chunk
#pragma unroll
  for (int sl = 0; sl < DT_SLOTS; sl++) {
    const int k = wave + sl * DT_NW;
    if (k >= K) continue;
    float *pk = partial + ((size_t)blockIdx.x * K + k) * (size_t)n_a * n_b;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int c = ct * DT_T + 2 * (4 * g + r) + i;
        if (c >= n_a) continue;
        if (cb + 0 < n_b) pk[(size_t)c * n_b + cb + 0] = acc[sl][i][0][r];
        if (cb + 1 < n_b) pk[(size_t)c * n_b + cb + 1] = acc[sl][i][1][r];
      }
  }
}

// Wider layers: a wavefront per (tap, 64 x 64 channel tile, share of the positions), no LDS; a
// workgroup holds the 2 x 2 tiles of a 128 x 128 block and keeps them in step with a barrier
// per granule, so that of the two wavefronts that need the same quads the second reads L1 (the
// kernel is bound by the traffic between L2 and the compute units: 512 bytes per position and
// tile for 64 MFMAs).
// As in k_conv_dw_taps the MFMA contracts over four positions and the operands come straight
// from the rows: lane (r, g) loads the four channels 4 r .. 4 r + 3 of position 4 g + kk (16
// lanes read 256 consecutive bytes); the sixteen instructions of a position quad pair component
// i of the a-side with component j of the b-side, so instruction (i, j) computes rows
// 4 * (MFMA row) + i and columns 4 * (MFMA column) + j of the tile.
// Granules without the tap are skipped by the granule masks (when the table has them).  A tap
// with few rules gets few shares (tap_shares, from the table's rule counts) so that every
// wavefront carries about the same number of rules, and only those shares' partial results are
// written and summed (k_sum_shares); blocks of DT_BLOCK granules are dealt
// round-robin over a tap's shares.  The loop runs two granules ahead: while the MFMAs of one
// granule issue, the rows of the next are on their way and the indices of the one after.
constexpr int DWV_T = 64;
struct TapShares {
  unsigned short n[32];  // K <= 32: shares of tap k that have work; the rest neither run nor are summed
};
// k_sum_blocks over the partial results of k_conv_dw_wave: output i belongs to tap i / per_tap,
// whose first tap_shares.n[tap] blocks hold sums (all `blocks` of them when K > 32).  Same fixed order.
__global__ __launch_bounds__(1024) void k_sum_shares(const float *__restrict__ partial, int blocks, int64_t stride,
                                                     int64_t count, int per_tap, int K, TapShares tap_shares,
                                                     float *__restrict__ out) {
  __shared__ float part[16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t i = (int64_t)blockIdx.x * 64 + lane;
  const int waves = blockDim.x >> 6;
  float s = 0;
  if (i < count) {
    const int mine = K <= 32 ? min(blocks, (int)tap_shares.n[i / per_tap]) : blocks;
    const int per = (mine + waves - 1) / waves;
    const int b0 = min(mine, wave * per), b1 = min(mine, b0 + per);
#pragma unroll 4
    for (int b = b0; b < b1; b++) s += partial[(size_t)b * stride + i];
  }
  part[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && i < count) {
    float tot = 0;
    for (int w = 0; w < waves; w++) tot += part[w][lane];
    out[i] = tot;
  }
}
// NA, NB: channels per lane on the a- and the b-side (4; 2 for a side of at most 32 channels; 3 where
// tiles of 48 channels leave fewer empty columns than tiles of 64, e.g. 96 = 2 x 48: a tile is
// 16 NA x 16 NB channels, and the MFMAs of a tile's empty part multiply zeros).
// VEC: a lane's channels come as one 16- or 8-byte load (plane counts multiples of NA / NB, arrays aligned).
template <bool VEC, int NA, int NB>
__global__ __launch_bounds__(256) void k_conv_dw_wave(const int *__restrict__ nbr, const int *__restrict__ rowmap,
                                                      const unsigned *__restrict__ gmask, int K, int64_t n, int64_t npad,
                                                      const float *__restrict__ a, int n_a, unsigned a_bytes,
                                                      const float *__restrict__ b, int n_b, unsigned b_bytes, int shares,
                                                      TapShares tap_shares, float *__restrict__ partial) {
  const int k = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // The four wavefronts of a workgroup: the 2 x 2 tiles of a 128 x 128 block, in step (see the
  // barriers below).  A layer of fewer than four tiles (at most 64 channels on one side and 128 on
  // the other) would leave wavefronts idle that way: there the workgroup's four wavefronts are
  // four (share, tile) pairs in a row, each on its own.
  constexpr int TA = 16 * NA, TB_ = 16 * NB;  // tile: TA channels of a by TB_ channels of b
  const int tiles_a = (n_a + TA - 1) / TA, tiles_b = (n_b + TB_ - 1) / TB_;
  const bool single = tiles_a * tiles_b < 4;
  const int slot = blockIdx.y * 4 + wave;
  const int share = single ? slot / (tiles_a * tiles_b) : blockIdx.y;
  const int tile = slot % (tiles_a * tiles_b);
  const int mt_o = (n_b + 2 * TB_ - 1) / (2 * TB_);
  const int ct = single ? tile / tiles_b : 2 * (blockIdx.z / mt_o) + (wave >> 1);
  const int ot = single ? tile % tiles_b : 2 * (blockIdx.z % mt_o) + (wave & 1);
  if (share >= shares) return;  // (single only: its wavefronts meet at no barrier)
  const int r16 = lane & 15, g = lane >> 4;
  const int ca = ct * TA + NA * r16, cb = ot * TB_ + NB * r16;
  const unsigned nowhere = 0x80000000u;  // offsets from here on read zeros
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a), 0, (int)a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(b), 0, (int)b_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t nbr_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<int *>(nbr), 0, (int)((unsigned)K * (unsigned)npad * 4u), 0x00020000);
  const __amdgpu_buffer_rsrc_t map_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<int *>(rowmap ? rowmap : nbr), 0, (int)((unsigned)npad * 4u), 0x00020000);
  const unsigned a_row_bytes = (unsigned)n_a * 4u, b_row_bytes = (unsigned)n_b * 4u;
  // N channels of row j from column c0 on (negative row, or columns past the last: zeros)
  auto comps_of = [&](auto n_tag, const __amdgpu_buffer_rsrc_t &rsrc, int j, unsigned row_bytes, int c0, int width,
                      float *e) {
    constexpr int N = decltype(n_tag)::value;
    const unsigned row = (unsigned)j * row_bytes;
    if constexpr (VEC && N == 4) {
      const unsigned off = (j < 0 || c0 >= width) ? nowhere : row + (unsigned)c0 * 4u;
      const v4f v = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0));
      e[0] = v.x, e[1] = v.y, e[2] = v.z, e[3] = v.w;
    } else if constexpr (VEC && N == 3) {
      const unsigned off = (j < 0 || c0 >= width) ? nowhere : row + (unsigned)c0 * 4u;
      const v3f v = __builtin_bit_cast(v3f, __builtin_amdgcn_raw_buffer_load_b96(rsrc, off, 0, 0));
      e[0] = v.x, e[1] = v.y, e[2] = v.z;
    } else if constexpr (VEC && N == 2) {
      const unsigned off = (j < 0 || c0 >= width) ? nowhere : row + (unsigned)c0 * 4u;
      const v2f v = __builtin_bit_cast(v2f, __builtin_amdgcn_raw_buffer_load_b64(rsrc, off, 0, 0));
      e[0] = v.x, e[1] = v.y;
    } else {
#pragma unroll
      for (int x = 0; x < N; x++) {
        const unsigned off = (j < 0 || c0 + x >= width) ? nowhere : row + (unsigned)(c0 + x) * 4u;
        e[x] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, off, 0, 0));
      }
    }
  };
  v4f acc[NA][NB];
#pragma unroll
  for (int i = 0; i < NA; i++)
#pragma unroll
    for (int j = 0; j < NB; j++) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  const int n_granules = (int)((n + 15) >> 4), n32 = (int)n;
  const bool idle = ct * TA >= n_a || ot * TB_ >= n_b;  // a tile past the last channel: only keeps the barrier count
  const int mine = K <= 32 ? (int)tap_shares.n[k] : shares;    // shares of this tap that have work
  if (share >= mine) return;  // uniform over the workgroup (over the wavefront when single); k_sum_shares does not read its part
  // This share's granules: blocks share, share + mine, ... of DT_BLOCK granules, those with the tap.
  // The masks of a block come as one pair of 16-byte loads (past the last granule they read zeros:
  // no tap) and are kept as a bit per granule, so that the search for the next granule with the
  // tap waits for memory once per block, not once per granule (the fine side of a filter = stride
  // rulebook has the tap in one granule of 2^dim).
  static_assert(DT_BLOCK == 8, "a block's granule masks are two 16-byte loads");
  const __amdgpu_buffer_rsrc_t gm_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<unsigned *>(gmask ? gmask : reinterpret_cast<const unsigned *>(nbr)), 0, (int)((unsigned)n_granules * 4u), 0x00020000);
  int cur_base = -DT_BLOCK;
  unsigned cur_bits = 0u;
  auto block_bits = [&](int base) {
    if (!gmask) return n_granules - base >= DT_BLOCK ? 0xFFu : (1u << (n_granules - base)) - 1u;
    const uint4 lo = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(gm_rsrc, (unsigned)base * 4u, 0, 0));
    const uint4 hi = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(gm_rsrc, (unsigned)base * 4u + 16u, 0, 0));
    const unsigned w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    unsigned bits = 0u;
#pragma unroll
    for (int i = 0; i < 8; i++) bits |= ((w[i] >> k) & 1u) << i;
    return bits;
  };
  auto seek = [&](int gi) {  // the first granule from gi on (a granule of one of the share's blocks) that has the tap
    for (;;) {
      if (gi >= n_granules) return n_granules;
      const int base = gi & ~(DT_BLOCK - 1);
      if (base != cur_base) cur_base = base, cur_bits = block_bits(base);
      const unsigned rem = cur_bits >> (gi & (DT_BLOCK - 1));
      if (rem) return gi + __builtin_ctz(rem);
      gi = base + mine * DT_BLOCK;
    }
  };
  auto next_granule = [&](int gi) {  // the one after gi (n_granules: none)
    if (gi >= n_granules) return n_granules;
    return seek((gi & (DT_BLOCK - 1)) == DT_BLOCK - 1 ? (gi & ~(DT_BLOCK - 1)) + mine * DT_BLOCK : gi + 1);
  };
  struct Quads {
    float a[4][NA], b[4][NB];
  };
  int4 jq, rq;  // neighbour rows and rows of b of the lane's four positions, for the granule whose rows are requested next
  auto load_indices = [&](int gi) {
    const unsigned toff = gi < n_granules ? (unsigned)(gi * 16 + 4 * g) * 4u : nowhere;
    jq = __builtin_bit_cast(int4, __builtin_amdgcn_raw_buffer_load_b128(nbr_rsrc, toff, (unsigned)k * (unsigned)npad * 4u, 0));
    const int t = gi * 16 + 4 * g;
    rq = make_int4(t, t + 1, t + 2, t + 3);
    if (rowmap) rq = __builtin_bit_cast(int4, __builtin_amdgcn_raw_buffer_load_b128(map_rsrc, toff, 0, 0));
  };
  auto load_rows = [&](int gi, Quads &q) {
    const int j[4] = {jq.x, jq.y, jq.z, jq.w}, r[4] = {rq.x, rq.y, rq.z, rq.w};
#pragma unroll
    for (int kk = 0; kk < 4; kk++) {
      const bool live = gi < n_granules && gi * 16 + 4 * g + kk < n32;
      comps_of(std::integral_constant<int, NA>(), a_rsrc, live ? j[kk] : -1, a_row_bytes, ca, n_a, q.a[kk]);
      comps_of(std::integral_constant<int, NB>(), b_rsrc, live ? r[kk] : -1, b_row_bytes, cb, n_b, q.b[kk]);
    }
  };
  auto multiply = [&](const Quads &q) {
#pragma unroll
    for (int kk = 0; kk < 4; kk++)
#pragma unroll
      for (int i = 0; i < NA; i++)
#pragma unroll
        for (int jx = 0; jx < NB; jx++)
          acc[i][jx] = __builtin_amdgcn_mfma_f32_16x16x4f32(q.a[kk][i], q.b[kk][jx], acc[i][jx], 0, 0, 0);
  };
  {
    Quads X, Y;
    int g0 = seek(share * DT_BLOCK);
    int g1 = next_granule(g0);
    if (!idle) {
      load_indices(g0);
      load_rows(g0, X);
      load_indices(g1);
    }
    while (g0 < n_granules) {
      // X: rows of g0 (requested), jq / rq: indices of g1 (requested).  The barriers keep the four
      // wavefronts on the same granule, so that of two that load the same quads one reads L1.
      const int g2 = next_granule(g1), g3 = next_granule(g2);
      if (!single) __syncthreads();
      if (!idle) {
        load_rows(g1, Y);
        load_indices(g2);
        multiply(X);
      }
      if (!single) __syncthreads();
      if (!idle) {
        load_rows(g2, X);
        load_indices(g3);
        if (g1 < n_granules) multiply(Y);
      }
      g0 = g2;
      g1 = g3;
    }
  }
  // acc[i][jx][r] = dW[k][ct*TA + NA (4 g + r) + i][ot*TB_ + NB r16 + jx] of this share (zeros for a share without work)
  float *pk = partial + ((size_t)share * K + k) * (size_t)n_a * n_b;
#pragma unroll
  for (int i = 0; i < NA; i++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int c = ct * TA + NA * (4 * g + r) + i;
      if (c >= n_a) continue;
#pragma unroll
      for (int jx = 0; jx < NB; jx++)
        if (cb + jx < n_b) pk[(size_t)c * n_b + cb + jx] = acc[i][jx][r];
    }
}

// Inputs of one to four channels (the first layer of a network: colour, occupancy): a tile of 16 a-side
// channels would be three quarters empty, so the 16 rows of the MFMA hold G = 16 / NA TAPS of NA
// channels each instead - lane (r, g) supplies channel r % NA of the row that tap m G + r / NA
// reads at position 4 g + kk - and NG such groups cover the filter (3 channels, 27 taps: 6 groups
// of 5 taps, 48 MFMAs per 16 positions where one tile per tap would issue 216).  A wavefront takes
// granules w, w + W, ... of the table for ALL taps (every wavefront sees every part of the
// pattern-sorted table; the rows of b are read once per granule), skips the groups none of whose
// taps the granule has, and runs two granules ahead like k_conv_dw_wave.  partial[w][K][NA][n_b].
template <int NA, int NG>
__global__ __launch_bounds__(256) void k_conv_dw_thin(const int *__restrict__ nbr, const int *__restrict__ rowmap,
                                                      const unsigned *__restrict__ gmask, int K, int64_t n, int64_t npad,
                                                      const float *__restrict__ a, unsigned a_bytes,
                                                      const float *__restrict__ b, int n_b, unsigned b_bytes,
                                                      float *__restrict__ partial) {
  constexpr int G = 16 / NA;
  const int lane = threadIdx.x & 63;
  const int w = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), W = gridDim.x * 4;
  const int r16 = lane & 15, g = lane >> 4;
  const int tsub = r16 / NA, chan = r16 % NA;
  const unsigned nowhere = 0x80000000u;  // offsets from here on read zeros
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a), 0, (int)a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(b), 0, (int)b_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t nbr_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<int *>(nbr), 0, (int)((unsigned)K * (unsigned)npad * 4u), 0x00020000);
  const __amdgpu_buffer_rsrc_t map_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<int *>(rowmap ? rowmap : nbr), 0, (int)((unsigned)npad * 4u), 0x00020000);
  // the lane's tap in group m, as the byte offset of its row of the table (nowhere: the lane holds
  // no tap there), and the taps of each group as a mask
  unsigned tap_off[NG], group_taps[NG];
#pragma unroll
  for (int m = 0; m < NG; m++) {
    const int tap = m * G + tsub;
    tap_off[m] = (tsub < G && tap < K) ? (unsigned)tap * (unsigned)npad * 4u : nowhere;
    group_taps[m] = (G >= 32 ? 0xFFFFFFFFu : ((1u << G) - 1u)) << (m * G);
  }
  const unsigned cb_off[2] = {r16 < n_b ? (unsigned)r16 * 4u : nowhere, 16 + r16 < n_b ? (unsigned)(16 + r16) * 4u : nowhere};
  const unsigned b_row_bytes = (unsigned)n_b * 4u;
  v4f acc[NG][2];
#pragma unroll
  for (int m = 0; m < NG; m++) acc[m][0] = acc[m][1] = (v4f){0.f, 0.f, 0.f, 0.f};
  const int n_granules = (int)((n + 15) >> 4), n32 = (int)n;
  struct Rows {
    float a[NG][4], b[4][2];
  };
  int4 jq[NG], rq;  // of the granule whose rows are requested next
  auto load_indices = [&](int gi) {
    const unsigned toff = gi < n_granules ? (unsigned)(gi * 16 + 4 * g) * 4u : nowhere;
#pragma unroll
    for (int m = 0; m < NG; m++)
      jq[m] = __builtin_bit_cast(int4, __builtin_amdgcn_raw_buffer_load_b128(
                                           nbr_rsrc, (toff | tap_off[m]) & nowhere ? nowhere : toff + tap_off[m], 0, 0));
    const int t = gi * 16 + 4 * g;
    rq = make_int4(t, t + 1, t + 2, t + 3);
    if (rowmap) rq = __builtin_bit_cast(int4, __builtin_amdgcn_raw_buffer_load_b128(map_rsrc, toff, 0, 0));
  };
  auto load_rows = [&](int gi, Rows &q) {
    const int r[4] = {rq.x, rq.y, rq.z, rq.w};
    bool live[4];
#pragma unroll
    for (int kk = 0; kk < 4; kk++) live[kk] = gi < n_granules && gi * 16 + 4 * g + kk < n32;
#pragma unroll
    for (int m = 0; m < NG; m++) {
      const int j[4] = {jq[m].x, jq[m].y, jq[m].z, jq[m].w};
#pragma unroll
      for (int kk = 0; kk < 4; kk++) {
        // a lane without a tap read zeros for its indices: row 0, which it must not gather
        const bool take = live[kk] && tap_off[m] != nowhere && j[kk] >= 0;
        q.a[m][kk] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                   a_rsrc, take ? (unsigned)j[kk] * (unsigned)(NA * 4) + (unsigned)chan * 4u : nowhere, 0, 0));
      }
    }
#pragma unroll
    for (int kk = 0; kk < 4; kk++)
#pragma unroll
      for (int nt = 0; nt < 2; nt++)
        q.b[kk][nt] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                    b_rsrc, (live[kk] && cb_off[nt] != nowhere) ? (unsigned)r[kk] * b_row_bytes + cb_off[nt] : nowhere, 0, 0));
  };
  auto taps_of = [&](int gi) {  // the taps granule gi has (wavefront-uniform)
    return (gmask && gi < n_granules) ? (unsigned)__builtin_amdgcn_readfirstlane((int)gmask[gi]) : 0xFFFFFFFFu;
  };
  auto multiply = [&](const Rows &q, unsigned present) {
#pragma unroll
    for (int m = 0; m < NG; m++) {
      if (!(present & group_taps[m])) continue;  // uniform over the wavefront
#pragma unroll
      for (int kk = 0; kk < 4; kk++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
          acc[m][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(q.a[m][kk], q.b[kk][nt], acc[m][nt], 0, 0, 0);
    }
  };
  {
    Rows X, Y;
    int g0 = min(w, n_granules), g1 = min(g0 + W, n_granules);
    unsigned p0 = taps_of(g0), p1 = taps_of(g1);
    load_indices(g0);
    load_rows(g0, X);
    load_indices(g1);
    while (g0 < n_granules) {
      // X: rows of g0 (requested), jq / rq: indices of g1 (requested)
      const int g2 = min(g1 + W, n_granules), g3 = min(g2 + W, n_granules);
      const unsigned p2 = taps_of(g2), p3 = taps_of(g3);
      load_rows(g1, Y);
      load_indices(g2);
      multiply(X, p0);
      load_rows(g2, X);
      load_indices(g3);
      if (g1 < n_granules) multiply(Y, p1);
      g0 = g2, g1 = g3, p0 = p2, p1 = p3;
    }
  }
  // acc[m][nt][r] = row 4 g + r of group m = (tap m G + (4 g + r) / NA, channel (4 g + r) % NA), column 16 nt + r16
  float *pw = partial + (size_t)w * K * NA * n_b;
#pragma unroll
  for (int m = 0; m < NG; m++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int row = 4 * g + r, tap = m * G + row / NA, c = row % NA;
      if (row >= G * NA || tap >= K) continue;
#pragma unroll
      for (int nt = 0; nt < 2; nt++)
        if (16 * nt + r16 < n_b) pw[((size_t)tap * NA + c) * n_b + 16 * nt + r16] = acc[m][nt][r];
    }
}

// Any groups, any shapes: one thread per weight, positions in order.  The correctness path for
// grouped convolutions, which the MFMA kernel does not cover.
__global__ void k_conv_dw_generic(const int *nbr, const int *rowmap, int K, int64_t n, int64_t npad, const float *a,
                                  int n_a, const float *b, int n_b, int groups, float *dw) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int ip = n_a / groups, op = n_b / groups;
  if (i >= (int64_t)K * groups * ip * op) return;
  const int o = (int)(i % op), c = (int)((i / op) % ip), g = (int)((i / ((int64_t)op * ip)) % groups);
  const int k = (int)(i / ((int64_t)op * ip * groups));
  float s = 0.f;
  for (int64_t t = 0; t < n; t++) {
    const int j = nbr[(int64_t)k * npad + t];
    if (j < 0) continue;
    const int64_t row = rowmap ? rowmap[t] : t;
    s += a[(int64_t)j * n_a + g * ip + c] * b[row * n_b + g * op + o];
  }
  dw[i] = s;
}

static void weight_gradient(Metadata &m, const Table &t, const float *a, int64_t a_rows, int n_a, const float *b,
                            int64_t b_rows, int n_b, int groups,
                            float *dw, hipStream_t s) {
  const int64_t per_chunk = (int64_t)t.K * (n_a / groups) * (n_b / groups) * groups;
  if (t.n == 0) {
    fill32(dw, 0, per_chunk, s);
    return;
  }
  if (groups != 1) {
    k_conv_dw_generic<<<grid_for(per_chunk), TB, 0, s>>>(t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, a, n_a, b, n_b,
                                                         groups, dw);
    LAUNCH_CHECK();
    return;
  }
  const bool vec4 = n_a % 4 == 0 && n_b % 4 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)b % 16 == 0;
  // one to four input channels: several taps share an MFMA's rows
  if (n_a <= 4 && n_b <= 32 && t.K <= 32 && t.npad % 4 == 0 && a_rows * n_a * 4 < ((int64_t)1 << 31) &&
      b_rows * n_b * 4 < ((int64_t)1 << 31) && (int64_t)t.K * t.npad * 4 < ((int64_t)1 << 31)) {
    const int groups_of_taps = (int)ceil_div(t.K, 16 / n_a);
    const int64_t n_granules = ceil_div(t.n, 16);
    const int64_t waves = round_up(std::min<int64_t>(n_granules, 2048), 4);
    const unsigned *gm = t.gmask.p;  // null when the table kept no granule masks
    bool done = true;
#define SCN_THIN(A, NGR)                                                                                            \
  k_conv_dw_thin<A, NGR><<<dim3((unsigned)(waves / 4)), 256, 0, s>>>(t.nbr.p, t.rowmap_ptr(), gm, t.K, t.n, t.npad, a, \
                                                                     (unsigned)(a_rows * n_a * 4), b, n_b,           \
                                                                     (unsigned)(b_rows * n_b * 4), m.partial.p)
    m.partial.reserve((size_t)waves * per_chunk);
    if (n_a == 3 && groups_of_taps <= 2) SCN_THIN(3, 2);
    else if (n_a == 3 && groups_of_taps <= 6) SCN_THIN(3, 6);
    else if (n_a == 1 && groups_of_taps <= 2) SCN_THIN(1, 2);
    else if (n_a == 4 && groups_of_taps <= 2) SCN_THIN(4, 2);
    else if (n_a == 4 && groups_of_taps <= 7) SCN_THIN(4, 7);
    else done = false;  // other shapes: the kernels below
#undef SCN_THIN
    if (done) {
      LAUNCH_CHECK();
      k_sum_blocks<float, float><<<dim3((unsigned)ceil_div(per_chunk, 64)), sum_threads(waves), 0, s>>>(m.partial.p, (int)waves, per_chunk, per_chunk, dw);
      LAUNCH_CHECK();
      return;
    }
  }
  // up to 32 channels on both sides; from there on the per-wavefront kernel below is faster
  // (64 -> 64 at 1 M sites: 1.97 against 1.3 ms)
  if (t.K <= DT_NW * DT_SLOTS && t.gmask.p && n_a <= DT_T && n_b <= DT_T && t.npad % 4 == 0 &&
      a_rows * n_a * 4 < ((int64_t)1 << 31) && b_rows * n_b * 4 < ((int64_t)1 << 31) &&
      (int64_t)t.K * t.npad * 4 < ((int64_t)1 << 31)) {
    // narrow layers: all taps per workgroup
    const int tiles = (int)(ceil_div(n_a, DT_T) * ceil_div(n_b, DT_T));
    // one resident round: two workgroups per compute unit, shared between the channel tiles
    const int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(ceil_div(t.n, 16 * DT_BLOCK), 512 / tiles));
    m.partial.reserve((size_t)chunks * per_chunk);
    const dim3 grid((unsigned)chunks, (unsigned)tiles);
    const bool vec2 = n_a % 2 == 0 && n_b % 2 == 0 && (uintptr_t)a % 8 == 0 && (uintptr_t)b % 8 == 0;
    if (vec2)
      k_conv_dw_taps<true><<<grid, DT_NW * 64, 0, s>>>(t.nbr.p, t.rowmap_ptr(), t.gmask.p, t.K, t.n, t.npad, a, n_a,
                                                       (unsigned)(a_rows * n_a * 4), b, n_b,
                                                       (unsigned)(b_rows * n_b * 4), m.partial.p);
    else
      k_conv_dw_taps<false><<<grid, DT_NW * 64, 0, s>>>(t.nbr.p, t.rowmap_ptr(), t.gmask.p, t.K, t.n, t.npad, a, n_a,
                                                        (unsigned)(a_rows * n_a * 4), b, n_b,
                                                       (unsigned)(b_rows * n_b * 4), m.partial.p);
    LAUNCH_CHECK();
    k_sum_blocks<float, float><<<dim3((unsigned)ceil_div(per_chunk, 64)), sum_threads(chunks), 0, s>>>(m.partial.p, (int)chunks, per_chunk, per_chunk, dw);
    LAUNCH_CHECK();
    return;
  }
  if (t.npad % 4 == 0 && a_rows * n_a * 4 < ((int64_t)1 << 31) && b_rows * n_b * 4 < ((int64_t)1 << 31) &&
      (int64_t)t.K * t.npad * 4 < ((int64_t)1 << 31) && t.K <= 65535) {
    // wider layers: a wavefront per (tap, 64 x 64 tile, share of the positions)
    // a side of at most 32 channels gives a lane two channels of it instead of four: tiles of 32 there
    // (a lane's three channels come as one 12-byte load: only with plane counts that are multiples of three)
    auto lane_channels = [](int planes) {
      if (planes <= 32) return 2;
      const int64_t pad4 = round_up(planes, 64), pad3 = round_up(planes, 48);
      return (planes % 3 == 0 && pad3 * 8 <= pad4 * 7) ? 3 : 4;
    };
    int na = lane_channels(n_a), nb = lane_channels(n_b);
    if (na == 3 && nb == 2) na = 4;  // the pairs of 3 and 2 are not built
    if (nb == 3 && na == 2) nb = 4;
    // one load per lane and side when the plane counts are multiples of the lane's channels and the
    // arrays aligned (16- and 8-byte loads to their size, 12-byte loads to a word)
    auto one_load = [&](int ka, int kb) {
      return n_a % ka == 0 && n_b % kb == 0 && (uintptr_t)a % (ka == 3 ? 4 : 4 * ka) == 0 &&
             (uintptr_t)b % (kb == 3 ? 4 : 4 * kb) == 0;
    };
    if (!one_load(na, nb)) na = na == 3 ? 4 : na, nb = nb == 3 ? 4 : nb;  // three channels per lane: as one load only
    const bool vec = one_load(na, nb);
    const int tile_a = 16 * na, tile_b = 16 * nb;
    const int tiles64 = (int)(ceil_div(n_a, tile_a) * ceil_div(n_b, tile_b));
    const bool single = tiles64 < 4;  // fewer than four tiles: a workgroup's wavefronts are (share, tile) pairs
    const int tiles = single ? 1 : (int)(ceil_div(n_a, 2 * tile_a) * ceil_div(n_b, 2 * tile_b));  // blocks of 2 x 2 tiles
    // Shares of the positions per tap in proportion to the tap's rules (the table's counts; the
    // first call on a table fetches them), about three workgroups per compute unit in all;
    // partial sums bounded to 256 MB, at least a block of granules per share.
    TapShares ts{};
    const int64_t groups_wanted = single ? 3072 / tiles64 : 768;  // shares of wavefronts, or workgroups of four tiles
    int64_t shares = ceil_div(groups_wanted, (int64_t)t.K * tiles);
    if (t.K <= 32 && t.K > 1) {
      ensure_counts(*t.cnt, s);
      int64_t most = 1, all = 0;
      for (int k = 0; k < t.K; k++) most = std::max(most, t.cnt->host[k]), all += t.cnt->host[k];
      shares = ceil_div(groups_wanted * most, std::max<int64_t>(1, all) * tiles);  // of the heaviest tap
    }
    shares = std::min<int64_t>(shares, std::max<int64_t>(1, ((int64_t)64 << 20) / per_chunk));
    shares = std::max<int64_t>(1, std::min<int64_t>(shares, ceil_div(t.n, 16 * DT_BLOCK)));
    if (t.K <= 32) {
      int64_t most = 1;
      for (int k = 0; k < t.K && t.K > 1; k++) most = std::max(most, t.cnt->host[k]);
      for (int k = 0; k < t.K; k++)
        ts.n[k] = (unsigned short)(t.K > 1 ? std::max<int64_t>(1, ceil_div(shares * t.cnt->host[k], most)) : shares);
    }
    if (tiles <= 65535 && shares <= 65535) {
      m.partial.reserve((size_t)shares * per_chunk);
      const dim3 grid((unsigned)t.K, (unsigned)(single ? ceil_div(shares * tiles64, 4) : shares), (unsigned)tiles);
      const unsigned *gm = (t.K <= 32 && t.gmask.p) ? t.gmask.p : nullptr;
#define SCN_DWV(V, A, B)                                                                                              \
  k_conv_dw_wave<V, A, B><<<grid, 256, 0, s>>>(t.nbr.p, t.rowmap_ptr(), gm, t.K, t.n, t.npad, a, n_a,                 \
                                               (unsigned)(a_rows * n_a * 4), b, n_b, (unsigned)(b_rows * n_b * 4),    \
                                               (int)shares, ts, m.partial.p)
      if (vec) {
        if (na == 4 && nb == 4) SCN_DWV(true, 4, 4);
        else if (na == 3 && nb == 3) SCN_DWV(true, 3, 3);
        else if (na == 3) SCN_DWV(true, 3, 4);
        else if (nb == 3) SCN_DWV(true, 4, 3);
        else if (na == 4) SCN_DWV(true, 4, 2);
        else if (nb == 4) SCN_DWV(true, 2, 4);
        else SCN_DWV(true, 2, 2);
      } else {
        if (na == 4 && nb == 4) SCN_DWV(false, 4, 4);
        else if (na == 4) SCN_DWV(false, 4, 2);
        else if (nb == 4) SCN_DWV(false, 2, 4);
        else SCN_DWV(false, 2, 2);
      }
#undef SCN_DWV
      LAUNCH_CHECK();
      k_sum_shares<<<dim3((unsigned)ceil_div(per_chunk, 64)), sum_threads(shares), 0, s>>>(m.partial.p, (int)shares, per_chunk, per_chunk,
                                                                                           n_a * n_b, t.K, ts, dw);
      LAUNCH_CHECK();
      return;
    }
  }
  const int tiles = (int)(ceil_div(n_a, DW_T) * ceil_div(n_b, DW_T));
  if (t.K > 65535 || tiles > 65535) throw Error("weight gradient: filter volume or channel count too large");
  // chunks: enough workgroups to fill the chip, partial sums bounded to about 256 MB
  int64_t chunks = ceil_div(2048, (int64_t)t.K * tiles);
  chunks = std::min<int64_t>(chunks, std::max<int64_t>(1, ((int64_t)64 << 20) / per_chunk));
  chunks = std::max<int64_t>(1, std::min<int64_t>(chunks, ceil_div(t.n, 4 * DW_PS)));
  const int64_t chunk_len = round_up(ceil_div(t.n, chunks), DW_PS);
  chunks = ceil_div(t.n, chunk_len);
  m.partial.reserve((size_t)chunks * per_chunk);
  const unsigned *gm = (t.K <= 32 && t.gmask.p) ? t.gmask.p : nullptr;
  const dim3 grid((unsigned)chunks, (unsigned)t.K, (unsigned)tiles);
  if (vec4)
    k_conv_dw<true><<<grid, 256, 0, s>>>(t.nbr.p, t.rowmap_ptr(), gm, t.K, t.n, t.npad, a, n_a, b, n_b, chunk_len,
                                         m.partial.p);
  else
    k_conv_dw<false><<<grid, 256, 0, s>>>(t.nbr.p, t.rowmap_ptr(), gm, t.K, t.n, t.npad, a, n_a, b, n_b, chunk_len,
                                          m.partial.p);
  LAUNCH_CHECK();
  k_sum_blocks<float, float><<<dim3((unsigned)ceil_div(per_chunk, 64)), sum_threads(chunks), 0, s>>>(m.partial.p, (int)chunks, per_chunk, per_chunk, dw);
  LAUNCH_CHECK();
}

// ---- input gradient when the rules cannot be read from the other side ----------------------------
// d_in[nbr[k][t]] += d_out[row(t)] * w[k]^T by scatter with atomics: submanifold rulebooks whose
// taps have no mirror image (even filter sizes) or whose level holds repeated points.  Correct
// for any table; the order of the additions, and so the last bits of the result, may vary.
__global__ void k_conv_dinput_scatter(const int *nbr, const int *rowmap, int K, int64_t n, int64_t npad,
                                      const float *d_out, const float *w, int n_in, int n_out, int groups,
                                      float *d_in) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * n_in) return;
  const int64_t t = i / n_in;
  const int c = (int)(i - t * n_in);
  const int ip = n_in / groups, op = n_out / groups, g = c / ip, cg = c - g * ip;
  const int64_t row = rowmap ? rowmap[t] : t;
  const float *d = d_out + row * n_out + g * op;
  for (int k = 0; k < K; k++) {
    const int j = nbr[(int64_t)k * npad + t];
    if (j < 0) continue;
    const float *wk = w + (((int64_t)k * groups + g) * ip + cg) * op;
    float acc = 0.f;
    for (int o = 0; o < op; o++) acc += d[o] * wk[o];
    atomicAdd(&d_in[(int64_t)j * n_in + c], acc);
  }
}
// flag[0] = 1 unless every position's centre tap names its own row (a level without repeated points)
__global__ void k_centre_is_identity(const int *nbr_centre, const int *rowmap, int64_t n, int *flag) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n && nbr_centre[t] != (rowmap ? rowmap[t] : (int)t)) flag[0] = 1;
}

// Whether rule (k, i -> j) of a submanifold table implies rule (K-1-k, j -> i): odd filter sizes
// on a level without repeated points.  Checked once per table (one host round trip).
static bool taps_mirror(Metadata &m, Table &t, const int64_t *filter, hipStream_t s) {
  if (t.mirror_known) return t.mirror;
  bool odd = true;
  for (int d = 0; d < m.dim; d++) odd = odd && (filter[d] % 2 == 1);
  t.mirror = odd;
  if (odd && t.n > 0) {
    m.dflags.reserve(16);
    fill32(m.dflags.p, 0, 1, s);
    k_centre_is_identity<<<grid_for(t.n), TB, 0, s>>>(t.nbr.p + (int64_t)(t.K / 2) * t.npad, t.rowmap_ptr(), t.n,
                                                      m.dflags.p);
    LAUNCH_CHECK();
    int flag = 0;
    HIP_CHECK(hipMemcpyAsync(&flag, m.dflags.p, sizeof(int), hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipStreamSynchronize(s));
    t.mirror = flag == 0;
  }
  t.mirror_known = true;
  return t.mirror;
}

// d_in = (table read from the output side) convolution of d_out with transposed weights.
static void input_gradient(Metadata &m, const Table &t, const float *d_out, int64_t d_out_rows, float *d_in,
                           const float *w, int n_in, int n_out, int groups, bool mirror, hipStream_t s) {
  const int64_t wn = (int64_t)t.K * (n_in / groups) * (n_out / groups) * groups;
  m.wt.reserve(wn);
  k_transpose_weights<<<grid_for(wn), TB, 0, s>>>(w, m.wt.p, t.K, groups, n_in / groups, n_out / groups, mirror ? 1 : 0);
  LAUNCH_CHECK();
  m.frozen = nullptr;  // the transposed weights are scratch of this call
  conv_forward(m, t, d_out, d_out_rows, d_in, m.wt.p, nullptr, n_out, n_in, groups, nullptr, nullptr, s);
}

// CPU/Convolution.cpp:152-185.  d_bias may be null.
void subm_conv_backward(Metadata &m, Table &t, const int64_t *filter, const float *in, float *d_in,
                        const float *d_out, const float *w, float *d_w, float *d_bias, int n_in, int n_out,
                        int groups, hipStream_t s) {
  if (groups < 1 || n_in < 1 || n_out < 1 || n_in % groups || n_out % groups)
    throw Error("channel counts must be positive multiples of groups");
  if (d_bias) column_sums(m, d_out, t.n, n_out, d_bias, s);
  weight_gradient(m, t, in, t.n, n_in, d_out, t.n, n_out, groups, d_w, s);
  if (t.n == 0) return;
  if (taps_mirror(m, t, filter, s)) {
    input_gradient(m, t, d_out, t.n, d_in, w, n_in, n_out, groups, true, s);
  } else {
    fill32(d_in, 0, t.n * n_in, s);
    k_conv_dinput_scatter<<<grid_for(t.n * n_in), TB, 0, s>>>(t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, d_out, w, n_in,
                                                               n_out, groups, d_in);
    LAUNCH_CHECK();
  }
}
// CPU/Convolution.cpp:81-115 (fwd: the table read from the coarse side, other: from the fine side)
// and CPU/Deconvolution.cpp:43-77 (fwd: from the fine side, other: from the coarse side).
// in_rows / out_rows: rows of the op's input and output levels.
void strided_conv_backward(Metadata &m, const Table &fwd, const Table &other, int64_t in_rows, int64_t out_rows,
                           const float *in, float *d_in, const float *d_out, const float *w, float *d_w, float *d_bias,
                           int n_in, int n_out, int groups, hipStream_t s) {
  if (groups < 1 || n_in < 1 || n_out < 1 || n_in % groups || n_out % groups)
    throw Error("channel counts must be positive multiples of groups");
  if (d_bias) {
    if (in_rows > 0)  // CPU/Convolution.cpp:98: only when the input level has rows
      column_sums(m, d_out, out_rows, n_out, d_bias, s);
    else
      fill32(d_bias, 0, n_out, s);
  }
  weight_gradient(m, fwd, in, in_rows, n_in, d_out, out_rows, n_out, groups, d_w, s);
  if (in_rows == 0) return;
  if (other.n != in_rows) throw Error("internal: the rulebook's other side does not match the input level");
  input_gradient(m, other, d_out, out_rows, d_in, w, n_in, n_out, groups, false, s);
}

// ---- batch normalisation, training mode ----------------------------------------------------------
// CPU/BatchNormalization.cpp:19-40: batch mean and biased variance into save_mean / save_invstd,
// running statistics updated with `momentum` weighting the old value and the unbiased variance;
// coef = scale | shift for the affine pass.
__global__ __launch_bounds__(1024) void k_bn_train_finish(const float *partial, int blocks, int planes, int64_t rows,
                                                          float *save_mean, float *save_invstd, float *running_mean,
                                                          float *running_var, const float *gamma, const float *beta,
                                                          float eps, float momentum, float *coef) {
  double s1, s2;
  pair_sums64(partial, blocks, planes, s1, s2);
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  if (threadIdx.x >= 64 || c >= planes) return;
  const double mean = s1 / (double)rows;
  double ss = s2 - mean * mean * (double)rows;  // sum of squared deviations
  if (ss < 0) ss = 0;
  save_mean[c] = (float)mean;
  running_mean[c] = momentum * running_mean[c] + (1 - momentum) * (float)mean;
  running_var[c] = momentum * running_var[c] + (1 - momentum) * (float)(ss / (double)(rows - 1));
  const float invstd = powf((float)(ss / (double)rows) + eps, -0.5f);
  save_invstd[c] = invstd;
  const float w = invstd * (gamma ? gamma[c] : 1.f);
  coef[c] = w;
  coef[planes + c] = -(float)mean * w + (beta ? beta[c] : 0.f);
}
// out = leaky(x * sc + sh), one thread per element (rows x planes), any strides
__global__ void k_affine_leaky(const float *in, float *out, int64_t rows, int planes, int64_t in_stride,
                               int64_t out_stride, const float *coef, float leak) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = rows * planes, step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const int64_t r = i / planes;
    const int c = (int)(i - r * planes);
    const float y = in[r * in_stride + c] * coef[c] + coef[planes + c];
    out[r * out_stride + c] = y * (y > 0 ? 1.f : leak);
  }
}
// The same, four planes per thread (plane count and strides multiples of four, 16-byte aligned).
__global__ void k_affine_leaky4(const float *__restrict__ in, float *__restrict__ out, int64_t rows, int planes,
                                int64_t in_stride, int64_t out_stride, const float *__restrict__ coef, float leak) {
  const int quads = planes >> 2;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = rows * quads, step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const int64_t r = i / quads;
    const int c = 4 * (int)(i - r * quads);
    const v4f x = *reinterpret_cast<const v4f *>(in + r * in_stride + c);
    const v4f sc = *reinterpret_cast<const v4f *>(coef + c), sh = *reinterpret_cast<const v4f *>(coef + planes + c);
    v4f y = x * sc + sh;
    y.x *= y.x > 0 ? 1.f : leak;
    y.y *= y.y > 0 ? 1.f : leak;
    y.z *= y.z > 0 ? 1.f : leak;
    y.w *= y.w > 0 ? 1.f : leak;
    *reinterpret_cast<v4f *>(out + r * out_stride + c) = y;
  }
}
void bn_train_forward(Metadata *scratch, const float *in, float *out, int64_t rows, int planes, int64_t in_stride,
                      int64_t out_stride, float *save_mean, float *save_invstd, float *running_mean,
                      float *running_var, const float *gamma, const float *beta, float eps, float momentum,
                      float leak, hipStream_t s) {
  if (planes <= 0) return;
  if (rows <= 0) {  // no rows: defined statistics (the reference divides by zero here), running ones untouched
    fill32(save_mean, 0, planes, s);
    fill32(save_invstd, 0, planes, s);
    return;
  }
  Metadata &m = *scratch;
  const ColsumPlan p = colsum_plan(rows, planes);
  m.partial.reserve((size_t)p.blocks * 2 * planes);
  m.prebuf.reserve(2 * (size_t)planes);
  launch_colsum<1>(dim3(p.blocks, (unsigned)ceil_div(planes, p.CW)), s, in, in_stride, nullptr, nullptr, 0, nullptr,
                                                                                 0.f, rows, planes, p.CW, p.rows_per_block,
                                                                                 m.partial.p);
  k_bn_train_finish<<<dim3((unsigned)ceil_div(planes, 64)), 1024, 0, s>>>(m.partial.p, p.blocks, planes, rows, save_mean,
                                                                          save_invstd, running_mean, running_var, gamma,
                                                                          beta, eps, momentum, m.prebuf.p);
  LAUNCH_CHECK();
  if (planes % 4 == 0 && in_stride % 4 == 0 && out_stride % 4 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0) {
    const int64_t blocks4 = std::min<int64_t>(ceil_div(rows * (planes / 4), TB), 256 * 64);
    k_affine_leaky4<<<dim3((unsigned)blocks4), TB, 0, s>>>(in, out, rows, planes, in_stride, out_stride, m.prebuf.p, leak);
    LAUNCH_CHECK();
    return;
  }
  const int64_t blocks = std::min<int64_t>(ceil_div(rows * planes, TB), 256 * 64);
  k_affine_leaky<<<dim3((unsigned)blocks), TB, 0, s>>>(in, out, rows, planes, in_stride, out_stride, m.prebuf.p, leak);
  LAUNCH_CHECK();
}
// CPU/BatchNormalization.cpp:84-106: coef = gradMean | k | invstd * gamma
__global__ __launch_bounds__(1024) void k_bn_bwd_finish(const float *partial, int blocks, int planes, int64_t rows,
                                                        const float *save_invstd, const float *gamma, float *d_gamma,
                                                        float *d_beta, float *coef) {
  double sd, dotp;
  pair_sums64(partial, blocks, planes, sd, dotp);
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  if (threadIdx.x >= 64 || c >= planes) return;
  const float invstd = save_invstd[c];
  if (d_beta) d_beta[c] = (float)sd;
  if (d_gamma) d_gamma[c] = (float)dotp * invstd;
  coef[c] = (float)(sd / (double)rows);
  coef[planes + c] = (float)dotp * invstd * invstd / (float)rows;
  coef[2 * planes + c] = invstd * (gamma ? gamma[c] : 1.f);
}
__global__ void k_bn_bwd_apply(const float *in, float *d_in, const float *out, const float *d_out, int64_t rows,
                               int planes, int64_t in_stride, int64_t out_stride, const float *save_mean,
                               const float *coef, float leak) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = rows * planes, step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const int64_t r = i / planes;
    const int c = (int)(i - r * planes);
    float d = d_out[r * out_stride + c];
    d *= out[r * out_stride + c] > 0.f ? 1.f : leak;
    d_in[r * in_stride + c] =
        (d - coef[c] - (in[r * in_stride + c] - save_mean[c]) * coef[planes + c]) * coef[2 * planes + c];
  }
}
// The same, four planes per thread (plane count and strides multiples of four, arrays 16-byte aligned).
__global__ void k_bn_bwd_apply4(const float *__restrict__ in, float *__restrict__ d_in, const float *__restrict__ out,
                                const float *__restrict__ d_out, int64_t rows, int planes, int64_t in_stride,
                                int64_t out_stride, const float *__restrict__ save_mean, const float *__restrict__ coef,
                                float leak) {
  const int quads = planes >> 2;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = rows * quads, step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const int64_t r = i / quads;
    const int c = 4 * (int)(i - r * quads);
    const v4f d = *reinterpret_cast<const v4f *>(d_out + r * out_stride + c);
    const v4f y = *reinterpret_cast<const v4f *>(out + r * out_stride + c);
    const v4f x = *reinterpret_cast<const v4f *>(in + r * in_stride + c);
    const v4f mu = *reinterpret_cast<const v4f *>(save_mean + c), c0 = *reinterpret_cast<const v4f *>(coef + c),
              c1 = *reinterpret_cast<const v4f *>(coef + planes + c), c2 = *reinterpret_cast<const v4f *>(coef + 2 * planes + c);
    v4f g;
    g.x = d.x * (y.x > 0.f ? 1.f : leak);
    g.y = d.y * (y.y > 0.f ? 1.f : leak);
    g.z = d.z * (y.z > 0.f ? 1.f : leak);
    g.w = d.w * (y.w > 0.f ? 1.f : leak);
    v4f o;
    o.x = (g.x - c0.x - (x.x - mu.x) * c1.x) * c2.x;
    o.y = (g.y - c0.y - (x.y - mu.y) * c1.y) * c2.y;
    o.z = (g.z - c0.z - (x.z - mu.z) * c1.z) * c2.z;
    o.w = (g.w - c0.w - (x.w - mu.w) * c1.w) * c2.w;
    *reinterpret_cast<v4f *>(d_in + r * in_stride + c) = o;
  }
}
// CPU/BatchNormalization.cpp:63-107.  d_out is not modified (the reference scales it in place).
void bn_backward(Metadata *scratch, const float *in, float *d_in, const float *out, const float *d_out, int64_t rows,
                 int planes, int64_t in_stride, int64_t out_stride, const float *save_mean, const float *save_invstd,
                 const float *gamma, float *d_gamma, float *d_beta, float leak, hipStream_t s) {
  if (planes <= 0) return;
  if (rows <= 0) {
    if (d_gamma) fill32(d_gamma, 0, planes, s);
    if (d_beta) fill32(d_beta, 0, planes, s);
    return;
  }
  Metadata &m = *scratch;
  const ColsumPlan p = colsum_plan(rows, planes);
  m.partial.reserve((size_t)p.blocks * 2 * planes);
  m.prebuf.reserve(3 * (size_t)planes);
  launch_colsum<2>(dim3(p.blocks, (unsigned)ceil_div(planes, p.CW)), s, in, in_stride, d_out, out, out_stride,
                                                                                 save_mean, leak, rows, planes, p.CW,
                                                                                 p.rows_per_block, m.partial.p);
  k_bn_bwd_finish<<<dim3((unsigned)ceil_div(planes, 64)), 1024, 0, s>>>(m.partial.p, p.blocks, planes, rows, save_invstd,
                                                                        gamma, d_gamma, d_beta, m.prebuf.p);
  LAUNCH_CHECK();
  auto al = [](const float *p) { return (uintptr_t)p % 16 == 0; };
  if (planes % 4 == 0 && in_stride % 4 == 0 && out_stride % 4 == 0 && al(in) && al(d_in) && al(out) && al(d_out) &&
      al(save_mean)) {
    const int64_t blocks4 = std::min<int64_t>(ceil_div(rows * (planes / 4), TB), 256 * 64);
    k_bn_bwd_apply4<<<dim3((unsigned)blocks4), TB, 0, s>>>(in, d_in, out, d_out, rows, planes, in_stride, out_stride,
                                                           save_mean, m.prebuf.p, leak);
    LAUNCH_CHECK();
    return;
  }
  const int64_t blocks = std::min<int64_t>(ceil_div(rows * planes, TB), 256 * 64);
  k_bn_bwd_apply<<<dim3((unsigned)blocks), TB, 0, s>>>(in, d_in, out, d_out, rows, planes, in_stride, out_stride, save_mean,
                                                       m.prebuf.p, leak);
  LAUNCH_CHECK();
}

// ---- pooling -------------------------------------------------------------------------------------
// Gathers over the table read from the side of the gradient that is being written, one thread per
// (position, plane); taps in ascending order, as the reference walks its rule lists.
// MAX      CPU/MaxPooling.cpp:21-35,61-87: table = fine side; d_in[i][p] = sum over the windows o
//          that hold i of (out[o][p] == in[i][p] ? d_out[o][p] : 0).  The reference compares with
//          the input planes WITHOUT the nFeaturesToDrop offset its forward pass applies; so does this.
// AVERAGE  CPU/AveragePooling.cpp:21-35,62-86: table = fine side; d_in[i][drop + p] = sum of d_out[o][p] / K.
// UNPOOL   CPU/UnPooling.cpp:21-32,58-78: table = coarse side; d_in[o][drop + p] = sum of d_out[i][p].
// The columns of d_in the rules do not reach are zeroed.
enum { PB_MAX = 0, PB_AVERAGE = 1, PB_UNPOOL = 2 };
template <int MODE>
__global__ void k_pool_bwd(const int *nbr, const int *rowmap, int K, int64_t n, int64_t npad, const float *in,
                           float *d_in, int in_stride, const float *out, const float *d_out, int planes, int drop) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = n * in_stride, step = (int64_t)gridDim.x * blockDim.x;
  const int off = MODE == PB_MAX ? 0 : drop;
  for (; i < total; i += step) {
    const int64_t t = i / in_stride;
    const int col = (int)(i - t * in_stride);
    const int64_t row = rowmap ? rowmap[t] : t;
    const int p = col - off;
    float acc = 0.f;
    if (p >= 0 && p < planes) {
      const float x = MODE == PB_MAX ? in[row * in_stride + col] : 0.f;
      for (int k = 0; k < K; k++) {
        const int o = nbr[(int64_t)k * npad + t];
        if (o < 0) continue;
        const float d = d_out[(int64_t)o * planes + p];
        if (MODE == PB_MAX)
          acc += out[(int64_t)o * planes + p] == x ? d : 0.f;
        else if (MODE == PB_AVERAGE)
          acc += d / (float)K;
        else
          acc += d;
      }
    }
    d_in[row * in_stride + col] = acc;
  }
}
// The same with nothing dropped and plane counts that are multiples of four: one thread per
// (position, four planes), 16-byte accesses, and only the taps the position's granule has
// (gmask; a fine row of a size = stride pooling has one) are looked at.
template <int MODE>
__global__ void k_pool_bwd4(const int *__restrict__ nbr, const int *__restrict__ rowmap, const unsigned *__restrict__ gmask,
                            int K, int64_t n, int64_t npad, const float *__restrict__ in, float *__restrict__ d_in,
                            const float *__restrict__ out, const float *__restrict__ d_out, int planes) {
  const int quads = planes >> 2;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = n * quads, step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const int64_t t = i / quads;
    const int c = 4 * (int)(i - t * quads);
    const int64_t row = rowmap ? rowmap[t] : t;
    v4f x = (v4f){0.f, 0.f, 0.f, 0.f}, acc = x;
    if (MODE == PB_MAX) x = *reinterpret_cast<const v4f *>(in + row * planes + c);
    unsigned taps = gmask ? gmask[t >> 4] : (K >= 32 ? 0xFFFFFFFFu : (1u << K) - 1u);
    while (taps) {
      const int k = __ffs((int)taps) - 1;
      taps &= taps - 1u;
      const int o = nbr[(int64_t)k * npad + t];
      if (o < 0) continue;
      const v4f d = *reinterpret_cast<const v4f *>(d_out + (int64_t)o * planes + c);
      if (MODE == PB_MAX) {
        const v4f y = *reinterpret_cast<const v4f *>(out + (int64_t)o * planes + c);
        acc.x += y.x == x.x ? d.x : 0.f;
        acc.y += y.y == x.y ? d.y : 0.f;
        acc.z += y.z == x.z ? d.z : 0.f;
        acc.w += y.w == x.w ? d.w : 0.f;
      } else if (MODE == PB_AVERAGE) {
        acc.x += d.x / (float)K, acc.y += d.y / (float)K, acc.z += d.z / (float)K, acc.w += d.w / (float)K;
      } else {
        acc += d;
      }
    }
    *reinterpret_cast<v4f *>(d_in + row * planes + c) = acc;
  }
}
void pool_backward(int mode, const Table &t, const float *in, float *d_in, int in_stride, const float *out,
                   const float *d_out, int planes, int drop, hipStream_t s) {
  if (t.n == 0 || in_stride <= 0) return;
  auto al = [](const float *p) { return p == nullptr || (uintptr_t)p % 16 == 0; };
  if (drop == 0 && in_stride == planes && planes % 4 == 0 && t.K <= 32 && al(in) && al(d_in) && al(out) && al(d_out)) {
    const int64_t blocks4 = std::min<int64_t>(ceil_div(t.n * (planes / 4), TB), 256 * 64);
    const dim3 g4((unsigned)blocks4);
    const unsigned *gm = t.gmask.p;
    if (mode == PB_MAX)
      k_pool_bwd4<PB_MAX><<<g4, TB, 0, s>>>(t.nbr.p, t.rowmap_ptr(), gm, t.K, t.n, t.npad, in, d_in, out, d_out, planes);
    else if (mode == PB_AVERAGE)
      k_pool_bwd4<PB_AVERAGE><<<g4, TB, 0, s>>>(t.nbr.p, t.rowmap_ptr(), gm, t.K, t.n, t.npad, in, d_in, out, d_out, planes);
    else
      k_pool_bwd4<PB_UNPOOL><<<g4, TB, 0, s>>>(t.nbr.p, t.rowmap_ptr(), gm, t.K, t.n, t.npad, in, d_in, out, d_out, planes);
    LAUNCH_CHECK();
    return;
  }
  const int64_t blocks = std::min<int64_t>(ceil_div(t.n * in_stride, TB), 256 * 64);
  const dim3 g((unsigned)blocks);
  if (mode == PB_MAX)
    k_pool_bwd<PB_MAX><<<g, TB, 0, s>>>(t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, in, d_in, in_stride, out, d_out, planes, drop);
  else if (mode == PB_AVERAGE)
    k_pool_bwd<PB_AVERAGE><<<g, TB, 0, s>>>(t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, in, d_in, in_stride, out, d_out, planes, drop);
  else
    k_pool_bwd<PB_UNPOOL><<<g, TB, 0, s>>>(t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, in, d_in, in_stride, out, d_out, planes, drop);
  LAUNCH_CHECK();
}

// ---- sparse to dense -------------------------------------------------------------------------------
// CPU/SparseToDense.cpp:21-33,66-90: d_in[row][p] = d_out[sample][p][offset(site)].
__global__ void k_s2d_bwd(Geom g, const int *soa, int64_t n, int64_t npad, float *d_in, const float *d_out, int planes,
                          int64_t vol) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = n * planes, step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const int64_t r = i / planes;
    const int p = (int)(i - r * planes);
    int64_t off = 0;
    for (int d = 0; d < g.dim; d++) off = off * g.size[d] + soa[d * npad + r];
    const int b = soa[g.dim * npad + r];
    d_in[i] = d_out[((int64_t)b * planes + p) * vol + off];
  }
}
void s2d_backward(const Level &l, float *d_in, const float *d_out, int planes, hipStream_t s) {
  if (l.n == 0 || planes <= 0) return;
  int64_t vol = 1;
  for (int d = 0; d < l.g.dim; d++) vol *= l.g.size[d];
  const int64_t blocks = std::min<int64_t>(ceil_div(l.n * planes, TB), 256 * 64);
  k_s2d_bwd<<<dim3((unsigned)blocks), TB, 0, s>>>(l.g, l.coords.p, l.n, l.npad, d_in, d_out, planes, vol);
  LAUNCH_CHECK();
}

// CPU/NetworkInNetwork.cpp:24-47 over the one-tap identity table.
void nin_backward(Metadata &m, const Table &t, const float *in, float *d_in, const float *d_out, const float *w,
                  float *d_w, float *d_bias, int n_in, int n_out, hipStream_t s) {
  if (d_bias) column_sums(m, d_out, t.n, n_out, d_bias, s);
  weight_gradient(m, t, in, t.n, n_in, d_out, t.n, n_out, 1, d_w, s);
  if (t.n == 0) return;
  input_gradient(m, t, d_out, t.n, d_in, w, n_in, n_out, 1, false, s);
}

}  // namespace scn
