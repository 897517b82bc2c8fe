// Bandwidth-bound forward ops: eval batch-norm + leaky ReLU, max pooling, the input and
// output layers and sparse-to-dense.  Each is a single pass that reads its input once
// and writes its output once with 16-byte accesses where the row length allows.
#include "metadata.h"

namespace scn {

static const int TB = 256;

// ---- batch norm (eval) + leaky ReLU -----------------------------------------------------
// CPU/BatchNormalization.cpp:41-61: w = gamma / sqrt(var + eps), b = beta - mean * w,
// y = x * w + b, y *= (y > 0 ? 1 : leakiness).
template <int V>
__global__ void k_bn_eval(const float *in, float *out, int64_t rows, int planes, int64_t in_stride,
                          int64_t out_stride, const float *mean, const float *var, const float *gamma,
                          const float *beta, float eps, float leak) {
  // scale / shift of every plane once per workgroup (LDS), then a pure streaming pass:
  // thread -> (row, group of V planes); consecutive threads cover one row, then the next
  extern __shared__ float coef[];  // [planes] scale | [planes] shift
  for (int c = threadIdx.x; c < planes; c += blockDim.x) {
    const float w = (1.0f / sqrtf(var[c] + eps)) * (gamma ? gamma[c] : 1.0f);
    coef[c] = w;
    coef[planes + c] = -mean[c] * w + (beta ? beta[c] : 0.0f);
  }
  __syncthreads();
  const int groups = planes / V;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = rows * groups;
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const int64_t r = i / groups;
    const int p0 = (int)(i - r * groups) * V;
    float x[V];
    if (V == 4) {
      float4 t = *reinterpret_cast<const float4 *>(in + r * in_stride + p0);
      x[0] = t.x, x[1] = t.y, x[2] = t.z, x[3] = t.w;
    } else {
      for (int v = 0; v < V; v++) x[v] = in[r * in_stride + p0 + v];
    }
    for (int v = 0; v < V; v++) {
      const float y = x[v] * coef[p0 + v] + coef[planes + p0 + v];
      x[v] = y * (y > 0 ? 1.0f : leak);
    }
    if (V == 4) {
      *reinterpret_cast<float4 *>(out + r * out_stride + p0) = make_float4(x[0], x[1], x[2], x[3]);
    } else {
      for (int v = 0; v < V; v++) out[r * out_stride + p0 + v] = x[v];
    }
  }
}

void bn_eval_forward(const float *in, float *out, int64_t rows, int planes, int64_t in_stride,
                     int64_t out_stride, const float *mean, const float *var, const float *gamma,
                     const float *beta, float eps, float leak, hipStream_t s) {
  if (rows <= 0 || planes <= 0) return;
  if (planes > 8192) throw Error("batch norm: more than 8192 planes");
  bool vec = planes % 4 == 0 && in_stride % 4 == 0 && out_stride % 4 == 0 &&
             ((uintptr_t)in % 16 == 0) && ((uintptr_t)out % 16 == 0);
  int64_t total = rows * (vec ? planes / 4 : planes);
  int64_t blocks = std::min<int64_t>(ceil_div(total, TB), 256 * 64);
  if (vec)
    k_bn_eval<4><<<dim3((unsigned)blocks), TB, 2 * planes * sizeof(float), s>>>(in, out, rows, planes, in_stride, out_stride, mean,
                                                       var, gamma, beta, eps, leak);
  else
    k_bn_eval<1><<<dim3((unsigned)blocks), TB, 2 * planes * sizeof(float), s>>>(in, out, rows, planes, in_stride, out_stride, mean,
                                                       var, gamma, beta, eps, leak);
  LAUNCH_CHECK();
}

// Pooling over a neighbour table, one thread per (output position, group of V planes).
// MAX     CPU/MaxPooling.cpp:7-20,37-60: the output starts at zero, so the result is
//         max(0, inputs of the window).
// AVERAGE CPU/AveragePooling.cpp:7-20,38-61: sum over the window's active inputs of
//         in / filter volume (absent sites count as zeros), taps in ascending order as the
//         reference walks its rule lists.
// UNPOOL  CPU/UnPooling.cpp:7-20,34-57: sum of the rows the table lists (over the fine level's
//         table of a strided rulebook that is the copy of the one coarse row above each site).
enum { POOL_MAX = 0, POOL_AVERAGE = 1, POOL_UNPOOL = 2 };
template <int V, int MODE>
__global__ void k_pool(const int *nbr, const int *rowmap, const unsigned *gmask, int K, int64_t n_out, int64_t npad,
                       const float *in, int in_stride, float *out, int planes, int64_t per_wg) {
  const int groups = planes / V;
  const float volume = (float)K;
  const int64_t total = n_out * groups;
  // Unpooling: workgroups b, b + 8, ... run on one XCD and together take one contiguous eighth of
  // the positions (the grid is a multiple of eight), each workgroup a contiguous piece of it, so
  // that the coarse row above a site's 2^dim children is fetched into one L2 instead of eight
  // (102 -> 40 MB read at a million sites).  Pooling: workgroups take turns over the table, whose
  // positions are sorted by cost - contiguous ranges would give one XCD the expensive end.
  const bool ranges = MODE == POOL_UNPOOL;
  const int64_t wg = ranges ? (int64_t)(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3) : (int64_t)blockIdx.x;
  int64_t i = (ranges ? wg * per_wg : wg * blockDim.x) + threadIdx.x;
  const int64_t end = ranges ? min(total, (wg + 1) * per_wg) : total;
  const int64_t step = ranges ? (int64_t)blockDim.x : (int64_t)gridDim.x * blockDim.x;
  for (; i < end; i += step) {
    const int64_t o = i / groups;
    const int p = (int)(i - o * groups) * V;
    float acc[V];
    for (int v = 0; v < V; v++) acc[v] = 0.0f;
    // taps that no row of this 16-row granule has are skipped without a look at the table (the
    // fine side of a filter = stride rulebook has one tap per row, and the rows are sorted by it)
    const unsigned present = gmask ? gmask[o >> 4] : 0xFFFFFFFFu;
    for (int k = 0; k < K; k++) {
      if (gmask && !((present >> k) & 1u)) continue;
      const int j = nbr[(int64_t)k * npad + o];
      if (j >= 0) {
        const float *src = in + (int64_t)j * in_stride + p;
        float x[V];
        if (V == 4) {
          const float4 t = *reinterpret_cast<const float4 *>(src);
          x[0] = t.x, x[1] = t.y, x[2] = t.z, x[3] = t.w;
        } else {
          for (int v = 0; v < V; v++) x[v] = src[v];
        }
        for (int v = 0; v < V; v++) {
          if (MODE == POOL_MAX)
            acc[v] = acc[v] < x[v] ? x[v] : acc[v];
          else if (MODE == POOL_AVERAGE)
            acc[v] += x[v] / volume;
          else
            acc[v] += x[v];
        }
      }
    }
    const int64_t row = rowmap ? rowmap[o] : o;
    if (V == 4)
      *reinterpret_cast<float4 *>(out + row * planes + p) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    else
      for (int v = 0; v < V; v++) out[row * planes + p + v] = acc[v];
  }
}
template <int MODE>
static void pool_launch(const Table &t, const float *in, int in_stride, float *out, int planes, int drop,
                        hipStream_t s) {
  if (t.n == 0 || planes <= 0) return;
  const bool vec = planes % 4 == 0 && in_stride % 4 == 0 && drop % 4 == 0 && ((uintptr_t)in % 16 == 0) &&
                   ((uintptr_t)out % 16 == 0);
  int64_t total = t.n * (vec ? planes / 4 : planes);
  const int64_t blocks = round_up(std::min<int64_t>(ceil_div(total, TB), 256 * 64), 8);
  const int64_t per_wg = round_up(ceil_div(total, blocks), TB);  // elements a workgroup takes, in turns of TB
  const unsigned *gm = t.K <= 32 ? t.gmask.p : nullptr;  // null when the table kept no granule masks
  if (vec)
    k_pool<4, MODE><<<dim3((unsigned)blocks), TB, 0, s>>>(t.nbr.p, t.rowmap_ptr(), gm, t.K, t.n, t.npad, in + drop,
                                                          in_stride, out, planes, per_wg);
  else
    k_pool<1, MODE><<<dim3((unsigned)blocks), TB, 0, s>>>(t.nbr.p, t.rowmap_ptr(), gm, t.K, t.n, t.npad, in + drop,
                                                          in_stride, out, planes, per_wg);
  LAUNCH_CHECK();
}
void maxpool_forward(const Table &t, const float *in, int in_stride, float *out, int planes, int drop,
                     hipStream_t s) {
  pool_launch<POOL_MAX>(t, in, in_stride, out, planes, drop, s);
}
void avgpool_forward(const Table &t, const float *in, int in_stride, float *out, int planes, int drop,
                     hipStream_t s) {
  pool_launch<POOL_AVERAGE>(t, in, in_stride, out, planes, drop, s);
}
void unpool_forward(const Table &t, const float *in, int in_stride, float *out, int planes, int drop,
                    hipStream_t s) {
  pool_launch<POOL_UNPOOL>(t, in, in_stride, out, planes, drop, s);
}

// ---- input / output layers --------------------------------------------------------------
// CPU/IOLayers.cpp:11-29: out[row] = sum over the row's points, in input order, of
// mult * in[point], mult = 1/count for mode 4.  Modes 1 / 2 / 5 copy the one point
// the site lists.
__global__ void k_input_fwd(const int *sorted_idx, const int *run_start, const int *run_len,
                            const unsigned char *overwrite, int64_t n_out, int mode, const float *in, float *out,
                            int planes, int average) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t total = n_out * planes;
  int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    int64_t r = i / planes;
    int p = (int)(i - r * planes);
    int st = run_start[r], len = run_len[r];
    float acc = 0.0f;
    if (mode == 1 || mode == 2 || mode == 5) {
      acc += in[(int64_t)listed_point(sorted_idx, st, len, mode, overwrite) * planes + p];
    } else {
      float mult = (average && len > 0) ? 1.0f / (float)len : 1.0f;
      for (int q = 0; q < len; q++) acc += mult * in[(int64_t)sorted_idx[st + q] * planes + p];
    }
    out[i] = acc;
  }
}
// The same for plane counts that are multiples of four: one thread per (row, four planes), 16-byte
// accesses; a row's run and point indices are read once per four planes.
__global__ void k_input_fwd4(const int *__restrict__ sorted_idx, const int *__restrict__ run_start,
                             const int *__restrict__ run_len, const unsigned char *__restrict__ overwrite, int64_t n_out,
                             int mode, const float *__restrict__ in, float *__restrict__ out, int planes, int average) {
  const int quads = planes >> 2;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = n_out * quads, step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const int64_t r = i / quads;
    const int c = 4 * (int)(i - r * quads);
    const int st = run_start[r], len = run_len[r];
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (mode == 1 || mode == 2 || mode == 5) {
      const float4 x = *reinterpret_cast<const float4 *>(in + (int64_t)listed_point(sorted_idx, st, len, mode, overwrite) * planes + c);
      acc.x += x.x, acc.y += x.y, acc.z += x.z, acc.w += x.w;
    } else {
      const float mult = (average && len > 0) ? 1.0f / (float)len : 1.0f;
      for (int q = 0; q < len; q++) {
        const float4 x = *reinterpret_cast<const float4 *>(in + (int64_t)sorted_idx[st + q] * planes + c);
        acc.x += mult * x.x, acc.y += mult * x.y, acc.z += mult * x.z, acc.w += mult * x.w;
      }
    }
    *reinterpret_cast<float4 *>(out + r * planes + c) = acc;
  }
}
// The same for one to four planes (coordinates-and-colour inputs): one thread per row, so that
// a row's run and point indices are read once instead of once per plane.
template <int P>
__global__ void k_input_fwd_row(const int *__restrict__ sorted_idx, const int *__restrict__ run_start,
                                const int *__restrict__ run_len, const unsigned char *__restrict__ overwrite, int64_t n_out,
                                int mode, const float *__restrict__ in, float *__restrict__ out, int average) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= n_out) return;
  const int st = run_start[r], len = run_len[r];
  float acc[P];
#pragma unroll
  for (int p = 0; p < P; p++) acc[p] = 0.0f;
  if (mode == 1 || mode == 2 || mode == 5) {
    const float *src = in + (int64_t)listed_point(sorted_idx, st, len, mode, overwrite) * P;
#pragma unroll
    for (int p = 0; p < P; p++) acc[p] += src[p];
  } else {
    const float mult = (average && len > 0) ? 1.0f / (float)len : 1.0f;
    for (int q = 0; q < len; q++) {
      const float *src = in + (int64_t)sorted_idx[st + q] * P;
#pragma unroll
      for (int p = 0; p < P; p++) acc[p] += mult * src[p];
    }
  }
#pragma unroll
  for (int p = 0; p < P; p++) out[r * P + p] = acc[p];
}
void input_forward(const InputRules &r, const float *in, float *out, int planes, hipStream_t s) {
  if (r.mode < 0) throw Error("input layer rules have not been built");
  if (planes <= 0) return;
  if (r.mode == 0) {
    if (r.n_in)
      HIP_CHECK(hipMemcpyAsync(out, in, sizeof(float) * r.n_in * planes, hipMemcpyDeviceToDevice, s));
    return;
  }
  if (r.n_out == 0) return;
  const int average = r.mode == 4 ? 1 : 0;
  if (planes <= 4) {
    const dim3 grid((unsigned)ceil_div(r.n_out, TB));
#define SCN_ROW(P)                                                                                                  \
  k_input_fwd_row<P><<<grid, TB, 0, s>>>(r.sorted_idx.p, r.run_start.p, r.run_len.p, r.overwrite.p, r.n_out, r.mode, in, \
                                         out, average)
    if (planes == 1) SCN_ROW(1);
    else if (planes == 2) SCN_ROW(2);
    else if (planes == 3) SCN_ROW(3);
    else SCN_ROW(4);
#undef SCN_ROW
    LAUNCH_CHECK();
    return;
  }
  if (planes % 4 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0) {
    const int64_t blocks4 = std::min<int64_t>(ceil_div(r.n_out * (planes / 4), TB), 256 * 64);
    k_input_fwd4<<<dim3((unsigned)blocks4), TB, 0, s>>>(r.sorted_idx.p, r.run_start.p, r.run_len.p, r.overwrite.p, r.n_out,
                                                        r.mode, in, out, planes, average);
    LAUNCH_CHECK();
    return;
  }
  int64_t total = r.n_out * planes;
  int64_t blocks = std::min<int64_t>(ceil_div(total, TB), 256 * 64);
  k_input_fwd<<<dim3((unsigned)blocks), TB, 0, s>>>(r.sorted_idx.p, r.run_start.p, r.run_len.p, r.overwrite.p,
                                                    r.n_out, r.mode, in, out, planes, average);
  LAUNCH_CHECK();
}
// CPU/IOLayers.cpp:116-135 (and :207-229): the gradient of the output layer's input is
// InputLayer_ForwardPass without averaging: every site sums the gradients of the points it lists.
void output_backward(const InputRules &r, float *d_in, const float *d_out, int planes, hipStream_t s) {
  if (r.mode < 0) throw Error("input layer rules have not been built");
  if (planes <= 0) return;
  if (r.mode == 0) {
    if (r.n_in)
      HIP_CHECK(hipMemcpyAsync(d_in, d_out, sizeof(float) * r.n_in * planes, hipMemcpyDeviceToDevice, s));
    return;
  }
  if (r.n_out == 0) return;
  if (planes % 4 == 0 && (uintptr_t)d_out % 16 == 0 && (uintptr_t)d_in % 16 == 0) {
    const int64_t blocks4 = std::min<int64_t>(ceil_div(r.n_out * (planes / 4), TB), 256 * 64);
    k_input_fwd4<<<dim3((unsigned)blocks4), TB, 0, s>>>(r.sorted_idx.p, r.run_start.p, r.run_len.p, r.overwrite.p, r.n_out,
                                                        r.mode, d_out, d_in, planes, 0);
    LAUNCH_CHECK();
    return;
  }
  int64_t total = r.n_out * planes;
  int64_t blocks = std::min<int64_t>(ceil_div(total, TB), 256 * 64);
  k_input_fwd<<<dim3((unsigned)blocks), TB, 0, s>>>(r.sorted_idx.p, r.run_start.p, r.run_len.p, r.overwrite.p,
                                                    r.n_out, r.mode, d_out, d_in, planes, 0);
  LAUNCH_CHECK();
}

// CPU/IOLayers.cpp:95-115 (InputLayer_BackwardPass :31-47 without averaging): every input
// point listed in its site's rule receives the site's row; as a gather per input point.
// Modes 1 / 2 / 5 list a single point per site, the others get zeros.
// average != 0: the row is scaled by 1 / (number of points of the site), which makes this the
// gradient of the mode-4 input layer (CPU/IOLayers.cpp:31-47 with average = true).
template <int V>
__global__ void k_output_fwd(const int *row_of_input, const int *sorted_idx, const int *run_start,
                             const int *run_len, const unsigned char *overwrite, int64_t n_in, int mode,
                             const float *in, float *out, int planes, int average) {
  // thread -> (input point, group of V planes)
  const int groups = planes / V;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = n_in * groups;
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const int64_t pt = i / groups;
    const int p = (int)(i - pt * groups) * V;
    const int row = row_of_input[pt];
    bool listed = row >= 0;  // empty positions of a batch-by-length input get zeros
    if (listed && (mode == 1 || mode == 2 || mode == 5))
      listed = listed_point(sorted_idx, run_start[row], run_len[row], mode, overwrite) == (int)pt;
    const float mult = (average && listed) ? 1.0f / (float)run_len[row] : 1.0f;
    if (V == 4) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (listed) v = *reinterpret_cast<const float4 *>(in + (int64_t)row * planes + p);
      if (average) v = make_float4(mult * v.x, mult * v.y, mult * v.z, mult * v.w);
      *reinterpret_cast<float4 *>(out + pt * planes + p) = v;
    } else {
      const float v = listed ? in[(int64_t)row * planes + p] : 0.0f;
      out[pt * planes + p] = average ? mult * v : v;
    }
  }
}
static void output_forward_impl(const InputRules &r, const float *in, float *out, int planes, int average,
                                hipStream_t s) {
  if (r.mode < 0) throw Error("input layer rules have not been built");
  if (planes <= 0 || r.n_in == 0) return;
  if (r.mode == 0) {
    HIP_CHECK(hipMemcpyAsync(out, in, sizeof(float) * r.n_in * planes, hipMemcpyDeviceToDevice, s));
    return;
  }
  if (r.n_out == 0) {  // every position empty
    fill32(out, 0, r.n_in * planes, s);
    return;
  }
  const bool vec = planes % 4 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0;
  const int64_t total = r.n_in * (vec ? planes / 4 : planes);
  const int64_t blocks = std::min<int64_t>(ceil_div(total, TB), 256 * 64);
  if (vec)
    k_output_fwd<4><<<dim3((unsigned)blocks), TB, 0, s>>>(r.row_of_input.p, r.sorted_idx.p, r.run_start.p,
                                                          r.run_len.p, r.overwrite.p, r.n_in, r.mode, in, out, planes,
                                                          average);
  else
    k_output_fwd<1><<<dim3((unsigned)blocks), TB, 0, s>>>(r.row_of_input.p, r.sorted_idx.p, r.run_start.p,
                                                          r.run_len.p, r.overwrite.p, r.n_in, r.mode, in, out, planes,
                                                          average);
  LAUNCH_CHECK();
}
void output_forward(const InputRules &r, const float *in, float *out, int planes, hipStream_t s) {
  output_forward_impl(r, in, out, planes, 0, s);
}
// CPU/IOLayers.cpp:73-93 (and :161-184): every listed point receives its site's gradient, scaled
// by 1 / count in mode 4; points a site does not list, and empty positions, get zeros.
void input_backward(const InputRules &r, float *d_in, const float *d_out, int planes, hipStream_t s) {
  output_forward_impl(r, d_out, d_in, planes, r.mode == 4 ? 1 : 0, s);
}

// ---- sparse to dense --------------------------------------------------------------------
// CPU/SparseToDense.cpp:7-19,35-64: out[sample][plane][offset(site)] = in[row][plane] on a
// zero-filled [batch, planes, spatial...] tensor.
// One thread per (site, group of `pchunk` planes; 8 with 16-byte loads of the row), sites taken in the level's schedule (ascending
// site key): the lanes of a wavefront hold sites that are neighbours in space, so the 4-byte
// stores of one plane that fall into the same 32-byte sector leave as one write.
__global__ void k_s2d(Geom g, const int *__restrict__ soa, const int *__restrict__ sched, int64_t n, int64_t npad,
                      const float *__restrict__ in, float *__restrict__ out, int planes, int64_t vol, int pchunk, bool vec4) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const int64_t r = sched ? sched[t] : t;
  int64_t off = 0;
  for (int d = 0; d < g.dim; d++) off = off * g.size[d] + soa[d * npad + r];
  const int b = soa[g.dim * npad + r];
  const int p0 = blockIdx.y * pchunk, p1 = min(planes, p0 + pchunk);
  const float *src = in + r * planes;
  float *dst = out + (int64_t)b * planes * vol + off;
  if (vec4) {  // pchunk = 8 on 16-byte aligned rows: two loads, then the stores
    const float4 x0 = *reinterpret_cast<const float4 *>(src + p0);
    const float4 x1 = p0 + 4 < p1 ? *reinterpret_cast<const float4 *>(src + p0 + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
    const float v[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
    for (int i = 0; i < 8; i++)
      if (p0 + i < p1) dst[(int64_t)(p0 + i) * vol] = v[i];
    return;
  }
  for (int p = p0; p < p1; p++) dst[(int64_t)p * vol] = src[p];
}
void s2d_forward(const Level &l, const float *in, float *out, int planes, hipStream_t s) {
  int64_t vol = 1;
  for (int d = 0; d < l.g.dim; d++) vol *= l.g.size[d];
  fill32(out, 0, (int64_t)l.batch * planes * vol, s);
  if (l.n == 0 || planes <= 0) return;
  const bool vec4 = planes % 4 == 0 && (uintptr_t)in % 16 == 0;
  const int pchunk = vec4 ? 8 : 4;
  const dim3 grid((unsigned)ceil_div(l.n, TB), (unsigned)ceil_div(planes, pchunk));
  k_s2d<<<grid, TB, 0, s>>>(l.g, l.coords.p, l.sched_ptr(), l.n, l.npad, in, out, planes, vol, pchunk, vec4);
  LAUNCH_CHECK();
}

// ---- active pooling ------------------------------------------------------------------------
// CPU/ActivePooling.cpp:8-25,47-63: out[sample] = sum of the sample's rows (times 1 / count with
// average), out is [batch, planes].  The level's schedule lists rows by ascending site key and
// the sample index is the key's top part, so every sample is one contiguous range of schedule
// positions: start[b] .. start[b + 1].  Sums are taken in that order, in a fixed number of chunks
// per sample, then over the chunks: the same bits on every run.
__global__ void k_sample_starts(const int *soa, const int *sched, int dim, int64_t n, int64_t npad, int batch,
                                int *start) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const int *sample = soa + (int64_t)dim * npad;
  const int b = sample[sched ? sched[t] : t];
  const int before = t > 0 ? sample[sched ? sched[t - 1] : t - 1] : -1;
  for (int q = before + 1; q <= b; q++) start[q] = (int)t;  // samples without sites begin where the next one does
  if (t == n - 1)
    for (int q = b + 1; q <= batch; q++) start[q] = (int)n;
}
// grid (sample * chunks + chunk, column tile of CW): partial[(sample * chunks + chunk) * planes + c]
template <int V>
__global__ __launch_bounds__(256) void k_active_pool_partial(const int *__restrict__ sched, const int *__restrict__ start,
                                                             int n_one, int chunks, const float *__restrict__ in, int planes,
                                                             int CW, float *__restrict__ partial) {
  // A thread owns V consecutive planes (V = 4: 16-byte loads) and has four rows in flight.
  __shared__ float red[256 * V];
  const int b = blockIdx.x / chunks, chunk = blockIdx.x % chunks;
  const int TPR = CW / V;
  const int tx = threadIdx.x % TPR, ty = threadIdx.x / TPR, RW = 256 / TPR;
  const int c = blockIdx.y * CW + tx * V;
  // n_one >= 0: a level of one sample, all n_one rows are its rows (start is not read)
  const int lo = n_one >= 0 ? 0 : start[b], hi = n_one >= 0 ? n_one : start[b + 1];
  const int per = (hi - lo + chunks - 1) / chunks;
  const int t0 = min(hi, lo + chunk * per), t1 = min(hi, t0 + per);
  float acc[V];
#pragma unroll
  for (int v = 0; v < V; v++) acc[v] = 0.f;
  if (c < planes) {
    auto add_row = [&](int t) {
      const float *src = in + (int64_t)(sched ? sched[t] : t) * planes + c;
      if constexpr (V == 4) {
        const float4 x = *reinterpret_cast<const float4 *>(src);
        acc[0] += x.x, acc[1] += x.y, acc[2] += x.z, acc[3] += x.w;
      } else {
        acc[0] += src[0];
      }
    };
    int t = t0 + ty;
    for (; t + 3 * RW < t1; t += 4 * RW) {
      add_row(t);
      add_row(t + RW);
      add_row(t + 2 * RW);
      add_row(t + 3 * RW);
    }
    for (; t < t1; t += RW) add_row(t);
  }
#pragma unroll
  for (int v = 0; v < V; v++) red[threadIdx.x * V + v] = acc[v];
  __syncthreads();
  // red[(ty * TPR + tx) * V + v] = plane tx * V + v of row group ty: thread i < CW adds up plane i
  if (threadIdx.x < CW && blockIdx.y * CW + threadIdx.x < planes) {
    float sum = 0.f;
    for (int q = 0; q < RW; q++) sum += red[q * CW + threadIdx.x];
    partial[(size_t)blockIdx.x * planes + blockIdx.y * CW + threadIdx.x] = sum;
  }
}
// grid (sample, tile of 64 planes), 1024 threads: wavefront w adds up its contiguous share of the
// sample's chunks in order, wavefront 0 then the 16 shares in order (a fixed order).
__global__ __launch_bounds__(1024) void k_active_pool_finish(const float *__restrict__ partial, const int *__restrict__ start,
                                                             int n_one, int chunks, int batch, int planes, int average,
                                                             float *__restrict__ out) {
  __shared__ float part[16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int b = blockIdx.x, c = blockIdx.y * 64 + lane;
  const int per = (chunks + 15) / 16;
  const int q0 = min(chunks, wave * per), q1 = min(chunks, q0 + per);
  float s = 0.f;
  if (c < planes) {
    // eight loads in flight (one after the other, each waits out a trip to L2); the order of the
    // additions is fixed all the same
    int q = q0;
    for (; q + 8 <= q1; q += 8) {
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = partial[((size_t)b * chunks + q + i) * planes + c];
#pragma unroll
      for (int i = 0; i < 8; i++) s += v[i];
    }
    for (; q < q1; q++) s += partial[((size_t)b * chunks + q) * planes + c];
  }
  part[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && c < planes) {
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < 16; w++) tot += part[w][lane];
    const int count = n_one >= 0 ? n_one : start[b + 1] - start[b];
    out[(size_t)b * planes + c] = (average && count > 0) ? tot * (1.0f / (float)count) : tot;
  }
}
// CPU/ActivePooling.cpp:26-44,65-83: every row receives its sample's gradient.  A thread writes V
// consecutive planes of a row (V = 4: 16-byte accesses); n_one >= 0: a level of one sample with
// n_one rows (neither the sample column nor start is read).
template <int V>
__global__ void k_active_pool_bwd(const int *__restrict__ soa, int dim, int64_t n, int64_t npad,
                                  const int *__restrict__ start, int n_one, int planes, int average,
                                  const float *__restrict__ d_out, float *__restrict__ d_in) {
  const int groups = planes / V;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = n * groups, step = (int64_t)gridDim.x * blockDim.x;
  for (; i < total; i += step) {
    const int64_t r = i / groups;
    const int c = (int)(i - r * groups) * V;
    const int b = n_one >= 0 ? 0 : soa[(int64_t)dim * npad + r];
    const int count = n_one >= 0 ? n_one : start[b + 1] - start[b];
    const float mult = (average && count > 0) ? 1.0f / (float)count : 1.0f;
    const float *src = d_out + (int64_t)b * planes + c;
    float *dst = d_in + r * planes + c;
    if constexpr (V == 4) {
      const float4 x = *reinterpret_cast<const float4 *>(src);
      *reinterpret_cast<float4 *>(dst) = make_float4(x.x * mult, x.y * mult, x.z * mult, x.w * mult);
    } else {
      dst[0] = src[0] * mult;
    }
  }
}
static const int *sample_starts(Metadata &m, const Level &l, hipStream_t s) {
  m.s0.reserve(l.batch + 1);
  k_sample_starts<<<dim3((unsigned)ceil_div(l.n, TB)), TB, 0, s>>>(l.coords.p, l.sched_ptr(), l.g.dim, l.n, l.npad,
                                                                 l.batch, m.s0.p);
  LAUNCH_CHECK();
  return m.s0.p;
}
void active_pool_forward(Metadata &m, const Level &l, const float *in, float *out, int planes, int average,
                         hipStream_t s) {
  if (l.batch <= 0 || planes <= 0) return;
  if (l.n == 0) {
    fill32(out, 0, (int64_t)l.batch * planes, s);
    return;
  }
  // One sample: every row is its row, and the rows are added up as they lie in memory (any fixed
  // order gives the same bits on every run); several: by the schedule, where a sample's rows
  // are one range.
  const bool one = l.batch == 1;
  const int *start = one ? nullptr : sample_starts(m, l, s);
  const int *sched = one ? nullptr : l.sched_ptr();
  const int n_one = one ? (int)l.n : -1;
  // about a thousand workgroups over the batch, at least 256 rows each on average
  int chunks = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(1024, l.batch), ceil_div(l.n, (int64_t)256 * l.batch)));
  const int CW = planes <= 16 ? 16 : planes <= 32 ? 32 : 64;
  m.partial.reserve((size_t)l.batch * chunks * planes);
  const dim3 grid((unsigned)(l.batch * chunks), (unsigned)ceil_div(planes, CW));
  if (planes % 4 == 0 && (uintptr_t)in % 16 == 0)
    k_active_pool_partial<4><<<grid, 256, 0, s>>>(sched, start, n_one, chunks, in, planes, CW, m.partial.p);
  else
    k_active_pool_partial<1><<<grid, 256, 0, s>>>(sched, start, n_one, chunks, in, planes, CW, m.partial.p);
  LAUNCH_CHECK();
  k_active_pool_finish<<<dim3((unsigned)l.batch, (unsigned)ceil_div(planes, 64)), 1024, 0, s>>>(m.partial.p, start, n_one, chunks,
                                                                                              l.batch, planes, average, out);
  LAUNCH_CHECK();
}
void active_pool_backward(Metadata &m, const Level &l, float *d_in, const float *d_out, int planes, int average,
                          hipStream_t s) {
  if (l.n == 0 || planes <= 0) return;
  const bool one = l.batch == 1;
  const int *start = one ? nullptr : sample_starts(m, l, s);
  const int n_one = one ? (int)l.n : -1;
  const bool vec = planes % 4 == 0 && (uintptr_t)d_in % 16 == 0 && (uintptr_t)d_out % 16 == 0;
  const int64_t blocks = std::min<int64_t>(ceil_div(l.n * (vec ? planes / 4 : planes), TB), 256 * 64);
  if (vec)
    k_active_pool_bwd<4><<<dim3((unsigned)blocks), TB, 0, s>>>(l.coords.p, l.g.dim, l.n, l.npad, start, n_one, planes, average,
                                                               d_out, d_in);
  else
    k_active_pool_bwd<1><<<dim3((unsigned)blocks), TB, 0, s>>>(l.coords.p, l.g.dim, l.n, l.npad, start, n_one, planes, average,
                                                               d_out, d_in);
  LAUNCH_CHECK();
}

}  // namespace scn
