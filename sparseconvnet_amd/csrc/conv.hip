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
#include "conv_common.h"

#include <map>
#include <mutex>

namespace scn {

// ---- scratch of a convolution -------------------------------------------------------------------
// The kernels below need device memory beyond their inputs and outputs: the weights in MFMA
// operand order, the set counters of the resident-weights kernel, and partial tiles when a small
// level's taps are split over workgroups.  Normally these are buffers of the handle, grown on
// demand from the block cache.  The allocation-free entry point (scn_subm_conv_fwd_noalloc) may
// not allocate: it takes them from this array instead, one copy per GPU, held until the process
// ends and shared by every such call on that GPU (overlapping calls on one GPU race).
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

float *scratch_wpack(Metadata &m, size_t floats) {
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
int *scratch_queue(Metadata &m, hipStream_t s) {
  if (m.fixed_scratch) return reinterpret_cast<int *>(m.fixed_scratch);
  if (!m.queue_zeroed) {
    m.queue.reserve(9 * 32);
    fill32(m.queue.p, 0, 9 * 32, s);
    m.queue_zeroed = true;
  }
  return m.queue.p;
}
// Partial tiles for n_split workgroups per tile; with the static scratch n_split shrinks until
// they fit (1: no partial tiles at all).
float *scratch_partial(Metadata &m, int &n_split, int64_t split_stride_floats) {
  if (m.fixed_scratch) {
    const int64_t fit = (int64_t)(NOALLOC_PARTIAL_BYTES / sizeof(float)) / std::max<int64_t>(split_stride_floats, 1);
    n_split = (int)std::max<int64_t>(1, std::min<int64_t>(n_split, fit));
    return n_split > 1 ? reinterpret_cast<float *>(m.fixed_scratch + NOALLOC_QUEUE_BYTES + NOALLOC_WPACK_BYTES) : nullptr;
  }
  if (n_split <= 1) return nullptr;
  m.partial.reserve((size_t)n_split * split_stride_floats);
  return m.partial.p;
}

__global__ void k_coefs(CoefJobs jobs) { coef_jobs(jobs); }
// Hands the pending jobs to the launch being prepared (and forgets them).

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
  int64_t row = rowmap ? rowmap[t] : t;
  if (epi.out2) epi_second(epi, row, oc, acc);
  if (epi.sc) acc = epi_act(acc, epi.sc[oc], epi.sh[oc], epi.leak);
  out[row * (epi.out_stride ? epi.out_stride : n_out) + oc] = acc;
}

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

// out[rowmap[pos]][col] = epilogue(bias[col] + sum over splits of partial[split][pos][col]), the
// splits added in ascending order.  A thread takes four columns of one position and has eight
// splits' loads in flight at a time (one load per split in a plain loop paid a cache latency per
// split: 8 us for the 27 splits of a 150-site level).
__global__ void k_conv_reduce(const float *__restrict__ partial, int n_split, int64_t split_stride, int ld,
                              const int *__restrict__ rowmap, int64_t n, Epi epi, float *__restrict__ out, int n_out) {
  const int ld4 = ld >> 2;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * ld4) return;
  const int64_t pos = i / ld4;
  const int c0 = 4 * (int)(i - pos * ld4);
  if (c0 >= n_out) return;
  const float *src = partial + pos * ld + c0;
  v4f acc = (v4f){0.f, 0.f, 0.f, 0.f};
  int sp = 0;
  for (; sp + 8 <= n_split; sp += 8) {
    v4f v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = *reinterpret_cast<const v4f *>(src + (int64_t)(sp + j) * split_stride);
#pragma unroll
    for (int j = 0; j < 8; j++) acc += v[j];
  }
  for (; sp < n_split; sp++) acc += *reinterpret_cast<const v4f *>(src + (int64_t)sp * split_stride);
  const int64_t row = rowmap ? rowmap[pos] : pos;
  float *o = out + row * (epi.out_stride ? epi.out_stride : n_out) + c0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    if (c0 + j >= n_out) break;
    float v = acc[j] + (epi.bias ? epi.bias[c0 + j] : 0.0f);
    if (epi.out2) epi_second(epi, row, c0 + j, v);
    if (epi.sc) v = epi_act(v, epi.sc[c0 + j], epi.sh[c0 + j], epi.leak);
    o[j] = v;
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

void launch_pack_weights(const float *w, float *wp, int K, int n_in, int n_out, int n_slab, int SS, int NCB,
                         int slab_stride, CoefJobs jobs, bool as_bf16, hipStream_t s) {
  const int64_t packed = (int64_t)K * n_slab * slab_stride;
  k_pack_weights<<<dim3((unsigned)ceil_div(packed, 256)), 256, 0, s>>>(w, wp, K, n_in, n_out, n_slab, SS, NCB, slab_stride,
                                                                      jobs, as_bf16);
  LAUNCH_CHECK();
}
void launch_pack_weights_part(const float *w, float *wp, int K, int w_rows, int n_in_part, int n_out, int SS, int NCB,
                              int *queue, CoefJobs jobs, bool as_bf16, hipStream_t s) {
  const int64_t packed = (int64_t)K * SS * NCB * 256;
  k_pack_weights_part<<<dim3((unsigned)ceil_div(packed, 256)), 256, 0, s>>>(w, wp, K, w_rows, n_in_part, n_out, SS, NCB,
                                                                           queue, jobs, as_bf16);
  LAUNCH_CHECK();
}
void launch_pack_weights_c4(const float *w, float *wp, int K, int n_in, int n_out, int NCB, int *queue, CoefJobs jobs,
                            hipStream_t s) {
  const int packed = K * NCB * 64;
  k_pack_weights_c4<<<dim3((unsigned)ceil_div(packed, 256)), 256, 0, s>>>(w, wp, K, n_in, n_out, NCB, queue, jobs);
  LAUNCH_CHECK();
}
void launch_conv_reduce(const float *partial, int n_split, int64_t split_stride, int ld, const int *rowmap, int64_t n,
                        Epi epi, float *out, int n_out, hipStream_t s) {
  k_conv_reduce<<<dim3((unsigned)ceil_div(n * (ld / 4), 256)), 256, 0, s>>>(partial, n_split, split_stride, ld, rowmap, n, epi,
                                                                           out, n_out);
  LAUNCH_CHECK();
}

template <bool PRE>
static bool conv_mfma_paths(Metadata &m, const Table &t, const float *in, float *out, const float *w,
                            Epi epi, int n_in, int n_out, PreArgs pre, hipStream_t s) {
  if (!PRE && try_few(m, t, in, out, w, epi, n_in, n_out, s)) return true;
  if (!PRE && try_resident(m, t, in, out, w, epi, n_in, n_out, s)) return true;
  const bool vec4 = n_in % 4 == 0 && ((uintptr_t)in % 16 == 0);
  if (n_out <= 128 && t.K <= 1024 && conv_rows_dispatch(vec4, PRE, m, t, in, out, w, epi, n_in, n_out, pre, s)) return true;
  if (t.K <= 1024 && conv_tiled_dispatch(vec4, PRE, m, t, in, out, w, epi, n_in, n_out, pre, s)) return true;
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
  struct FrozenReset {  // a frozen set and an output stride serve one call
    Metadata &m;
    ~FrozenReset() {
      m.frozen = nullptr;
      m.next_out_stride = 0;
      m.next_out2 = nullptr;
      m.before_pack = nullptr;
      m.wkey_ptr = 0;
    }
  } frozen_reset{m};
  if (groups < 1 || n_in < 1 || n_out < 1 || n_in % groups || n_out % groups)
    throw Error("channel counts must be positive multiples of groups");
  m.last_kernel.clear();
  if (t.n == 0) return;
  if (m.fixed_scratch && (bn || post || groups != 1))
    throw Error("allocation-free convolution: plain convolutions with groups = 1 only");
  // wider layers run as column ranges over a copy of the weights that would have to be allocated
  if (m.fixed_scratch && n_out > 256)
    throw Error("allocation-free convolution: at most 256 output planes");
  Epi epi;
  epi.bias = bias;
  if (m.next_out_stride) {
    if (m.next_out_stride < n_out || m.next_out_stride > INT32_MAX) throw Error("output stride below the plane count");
    if (n_out > 256 || m.fixed_scratch) throw Error("output stride: at most 256 output planes, not with the allocation-free entry");
    epi.out_stride = (int)m.next_out_stride;
  }
  m.jobs = CoefJobs();
  m.cur_in_rows = n_in_rows;
  m.cur_in_base = in;
  FrozenParams *frozen = m.fixed_scratch ? nullptr : m.frozen;
  if (frozen) {
    frozen->last = s;
    frozen->last_known = true;
  }
  if (m.next_out2) {
    if (n_out > 256 || m.fixed_scratch || groups != 1 || m.next_out2_stride < n_out || m.next_out2_stride > INT32_MAX)
      throw Error("second output: groups = 1, at most 256 output planes, a stride of at least that, not with the allocation-free entry");
    DevBuf<float> &buf = frozen ? frozen->post2 : m.post2buf;
    buf.reserve(2 * (size_t)n_out);
    m.jobs.post2 = CoefJob{m.next_out2_bn[0], m.next_out2_bn[1], m.next_out2_bn[2], m.next_out2_bn[3], m.next_out2_eps,
                           n_out, n_out, buf.p, buf.p + n_out};
    epi.out2 = m.next_out2;
    epi.out2_stride = (int)m.next_out2_stride;
    epi.sc2 = buf.p;
    epi.sh2 = buf.p + n_out;
    epi.leak2 = m.next_out2_leak;
  }
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
    if (frozen->post2_done) m.jobs.post2 = CoefJob();
    if (m.jobs.post.n_pad || m.jobs.pre.n_pad || m.jobs.post2.n_pad) {
      k_coefs<<<dim3(1), 256, 0, s>>>(take_jobs(m));
      LAUNCH_CHECK();
    }
    frozen->post_done = frozen->post_done || post != nullptr;
    frozen->pre_done = frozen->pre_done || pre_fused;
    frozen->post2_done = frozen->post2_done || epi.out2 != nullptr;
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
      // the copy runs when a kernel packs from it: not when a frozen set already holds the packed range
      m.before_pack = [=] {
        k_take_columns<<<dim3((unsigned)ceil_div(rows_w * wc, 256)), 256, 0, s>>>(w, rows_w, n_out, c0, wc, dst);
        LAUNCH_CHECK();
      };
      m.wkey_ptr = (int64_t)(uintptr_t)(w + rows_w * c0);
      m.wkey_from = (int64_t)(uintptr_t)dst;
      m.wkey_c0 = c0;
      m.wkey_wc = wc;
      Epi e = epi;
      if (e.bias) e.bias += c0;
      if (e.sc) e.sc += c0, e.sh += c0;
      e.out_stride = n_out;
      ok = conv_mfma_paths<false>(m, t, src, out + c0, dst, e, n_in, wc, PreArgs(), s);
      m.before_pack = nullptr;
      m.wkey_ptr = 0;
      m.last_kernel += " +";  // the next range's kernel is appended
    }
    if (ok) return;
  }
  if (m.jobs.post.n_pad || m.jobs.post2.n_pad) {  // no packing launch on this path: fold the coefficients by themselves
    k_coefs<<<dim3(1), 256, 0, s>>>(take_jobs(m));
    LAUNCH_CHECK();
  }
  int64_t total = t.n * n_out;
  note_kernel(m, "generic", {{"groups", groups}});
  k_conv_generic<<<dim3((unsigned)ceil_div(total, 256)), 256, 0, s>>>(t.nbr.p, t.rowmap_ptr(), t.K, t.n, t.npad, src,
                                                                       out, w, epi, n_in, n_out, groups);
  LAUNCH_CHECK();
}

}  // namespace scn

