// Convolution forward, output-stationary: every output row accumulates, over the filter
// taps, the row its neighbour table names times that tap's weight slice, and is written
// exactly once (no atomics, no read-modify-write of the output, deterministic).
// One kernel family serves SubmanifoldConvolution, Convolution and Deconvolution
// (CPU/Convolution.cpp:45-79,117-150, CPU/Deconvolution.cpp:7-41); they differ only in
// the table they pass.
#include "metadata.h"

namespace scn {

// Generic kernel: any channel counts, any groups.  One thread per (position, out channel).
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

void conv_forward(const Table &t, const int *rowmap, const float *in, float *out, const float *w,
                  const float *bias, int n_in, int n_out, int groups, hipStream_t s) {
  if (groups < 1 || n_in % groups || n_out % groups) throw Error("channel counts must be multiples of groups");
  if (t.n == 0) return;
  int64_t total = t.n * n_out;
  k_conv_generic<<<dim3((unsigned)ceil_div(total, 256)), 256, 0, s>>>(t.nbr.p, rowmap, t.K, t.n, t.npad, in,
                                                                       out, w, bias, n_in, n_out, groups);
  LAUNCH_CHECK();
}

}  // namespace scn
