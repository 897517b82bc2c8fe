// C-ABI harness around the reference's own CPU sources, compiled where they
// lie (never copied): the two #includes below pull in
// <reference>/sparseconvnet/SCN/Metadata/Metadata.cpp and the CPU/*.cpp files
// through the -I path given by oracle/Makefile.
//
// TEST INFRASTRUCTURE ONLY.  The resulting oracle/_ref/libscn_ref.so is used to
// validate oracle/scn_oracle.cpp, to write the golden fixtures under
// tests/golden/, and as the "reference" flavour of the CPU baseline.  The
// entry points mirror oracle/scn_oracle.cpp's (prefix ref_ instead of orc_) so
// one Python wrapper drives both.

#include <torch/torch.h>

#define ENABLE_OPENMP YES
#include <omp.h>

#include "Metadata/Metadata.cpp"
template class Metadata<1>;
template class Metadata<2>;
template class Metadata<3>;
template class Metadata<4>;
template class Metadata<5>;
template class Metadata<6>;

#include "CPU/BatchNormalization.cpp"
#include "CPU/Convolution.cpp"
#include "CPU/Deconvolution.cpp"
#include "CPU/IOLayers.cpp"
#include "CPU/AveragePooling.cpp"
#include "CPU/MaxPooling.cpp"
#include "CPU/UnPooling.cpp"
#include "CPU/NetworkInNetwork.cpp"
#include "CPU/SparseToDense.cpp"
#include "CPU/ActivePooling.cpp"

#include <cstring>

namespace {

struct Handle {
  int dim;
  void *m;
  at::Tensor feats = torch::empty({0}, at::kFloat);  // what sparseconvnet/inputBatch.py:18 keeps beside its Metadata
};

at::Tensor lt(const int64_t *p, int n) {
  return torch::from_blob((void *)p, {n}, at::kLong).clone();
}
at::Tensor ft(const float *p, std::vector<int64_t> shape) {
  if (!p) return torch::empty({0}, at::kFloat);
  return torch::from_blob((void *)p, shape, at::kFloat);
}
void copy_out(const at::Tensor &t, float *out) {
  auto c = t.contiguous();
  std::memcpy(out, c.data_ptr<float>(), sizeof(float) * c.numel());
}

template <Int D>
RuleBook &rb_get(Metadata<D> &m, int kind, const int64_t *a, const int64_t *b, const int64_t *c,
                 const int64_t *d) {
  auto A = lt(a, D);
  if (kind == 0) {
    auto B = lt(b, D);
    return m.getSubmanifoldRuleBook(A, B, true);
  }
  if (kind == 1) {
    auto B = lt(b, D), C = lt(c, D), Dd = lt(d, D);
    return m.getRuleBook(A, B, C, Dd, true);
  }
  return m.getSparseToDenseRuleBook(A, true);
}

}  // namespace

#define DISPATCH(h, ...)                                     \
  switch (((Handle *)h)->dim) {                              \
  case 1: { constexpr Int D = 1; auto &m = *(Metadata<1> *)((Handle *)h)->m; __VA_ARGS__; } break; \
  case 2: { constexpr Int D = 2; auto &m = *(Metadata<2> *)((Handle *)h)->m; __VA_ARGS__; } break; \
  case 3: { constexpr Int D = 3; auto &m = *(Metadata<3> *)((Handle *)h)->m; __VA_ARGS__; } break; \
  case 4: { constexpr Int D = 4; auto &m = *(Metadata<4> *)((Handle *)h)->m; __VA_ARGS__; } break; \
  case 5: { constexpr Int D = 5; auto &m = *(Metadata<5> *)((Handle *)h)->m; __VA_ARGS__; } break; \
  case 6: { constexpr Int D = 6; auto &m = *(Metadata<6> *)((Handle *)h)->m; __VA_ARGS__; } break; \
  }

extern "C" {

void *ref_md_create(int dim) {
  Handle *h = new Handle{dim, nullptr};
  switch (dim) {
  case 1: h->m = new Metadata<1>(); break;
  case 2: h->m = new Metadata<2>(); break;
  case 3: h->m = new Metadata<3>(); break;
  case 4: h->m = new Metadata<4>(); break;
  case 5: h->m = new Metadata<5>(); break;
  case 6: h->m = new Metadata<6>(); break;
  default: delete h; return nullptr;
  }
  return h;
}
void ref_md_destroy(void *h) {
  DISPATCH(h, (void)D; delete &m);
  delete (Handle *)h;
}
int ref_input_layer(void *h, const int64_t *spatial, const int64_t *coords, int n, int ncols,
                    int batchSize, int mode) {
  int r = 0;
  DISPATCH(h, auto S = lt(spatial, D);
           auto C = torch::from_blob((void *)coords, {n, ncols}, at::kLong).clone();
           m.inputLayer(S, C, batchSize, mode); r = *m.inputNActive);
  return r;
}
void ref_input_rules_header(void *h, int *hdr) {
  DISPATCH(h, (void)D; for (int i = 0; i < 4; i++) hdr[i] = m.inputLayerRuleBook[0][i]);
}
void ref_input_rules(void *h, int *rows) {
  DISPATCH(h, (void)D; if (m.inputLayerRuleBook.size() > 1) std::memcpy(
                           rows, m.inputLayerRuleBook[1].data(),
                           m.inputLayerRuleBook[1].size() * sizeof(Int)));
}
int ref_nactive(void *h, const int64_t *spatial) {
  int r = 0;
  DISPATCH(h, auto S = lt(spatial, D); r = m.getNActive(S));
  return r;
}
int ref_batch_size(void *h, const int64_t *spatial) {
  int r = 0;
  DISPATCH(h, auto S = lt(spatial, D); r = m.getBatchSize(S));
  return r;
}
void ref_spatial_locations(void *h, const int64_t *spatial, int64_t *out) {
  DISPATCH(h, auto S = lt(spatial, D); auto t = m.getSpatialLocations(S);
           std::memcpy(out, t.data_ptr<long>(), sizeof(int64_t) * t.numel()));
}
int ref_rb_noffsets(void *h, int kind, const int64_t *a, const int64_t *b, const int64_t *c,
                    const int64_t *d) {
  int r = 0;
  DISPATCH(h, r = (int)rb_get<D>(m, kind, a, b, c, d).size());
  return r;
}
void ref_rb_counts(void *h, int kind, const int64_t *a, const int64_t *b, const int64_t *c,
                   const int64_t *d, int64_t *counts) {
  DISPATCH(h, auto &rb = rb_get<D>(m, kind, a, b, c, d);
           for (size_t k = 0; k < rb.size(); k++) counts[k] = (int64_t)rb[k].size() / 2);
}
void ref_rb_copy(void *h, int kind, const int64_t *a, const int64_t *b, const int64_t *c,
                 const int64_t *d, int k, int *pairs) {
  DISPATCH(h, auto &rb = rb_get<D>(m, kind, a, b, c, d);
           std::memcpy(pairs, rb[k].data(), rb[k].size() * sizeof(Int)));
}

double ref_subm_conv(void *h, const int64_t *spatial, const int64_t *filter, const float *in,
                     float *out, const float *w, const float *bias, int nIn, int nOut, int groups) {
  double macs = 0;
  DISPATCH(h, auto S = lt(spatial, D); auto F = lt(filter, D); Int n = m.getNActive(S);
           auto I = ft(in, {n, nIn}); auto O = torch::empty({0}, at::kFloat);
           auto W = ft(w, {F.prod().item<int64_t>(), groups, nIn / groups, nOut / groups});
           auto B = ft(bias, {nOut});
           macs = cpu_SubmanifoldConvolution_updateOutput<float, D>(S, F, m, I, O, W, B);
           copy_out(O, out));
  return macs;
}
double ref_conv(void *h, const int64_t *inSz, const int64_t *outSz, const int64_t *filter,
                const int64_t *stride, const float *in, float *out, const float *w,
                const float *bias, int nIn, int nOut, int groups) {
  double macs = 0;
  DISPATCH(h, auto IS = lt(inSz, D); auto OS = lt(outSz, D); auto F = lt(filter, D);
           auto St = lt(stride, D); Int n = m.getNActive(IS); auto I = ft(in, {n, nIn});
           auto O = torch::empty({0}, at::kFloat);
           auto W = ft(w, {F.prod().item<int64_t>(), groups, nIn / groups, nOut / groups});
           auto B = ft(bias, {nOut});
           macs = cpu_Convolution_updateOutput<float, D>(IS, OS, F, St, m, I, O, W, B);
           copy_out(O, out));
  return macs;
}
double ref_deconv(void *h, const int64_t *inSz, const int64_t *outSz, const int64_t *filter,
                  const int64_t *stride, const float *in, float *out, const float *w,
                  const float *bias, int nIn, int nOut, int groups) {
  double macs = 0;
  DISPATCH(h, auto IS = lt(inSz, D); auto OS = lt(outSz, D); auto F = lt(filter, D);
           auto St = lt(stride, D); Int n = m.getNActive(IS); auto I = ft(in, {n, nIn});
           auto O = torch::empty({0}, at::kFloat);
           auto W = ft(w, {F.prod().item<int64_t>(), groups, nIn / groups, nOut / groups});
           auto B = ft(bias, {nOut});
           macs = cpu_Deconvolution_updateOutput<float, D>(IS, OS, F, St, m, I, O, W, B);
           copy_out(O, out));
  return macs;
}
void ref_maxpool(void *h, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                 const int64_t *stride, const float *in, int inStride, float *out, int nPlanes,
                 int nFeaturesToDrop) {
  DISPATCH(h, auto IS = lt(inSz, D); auto OS = lt(outSz, D); auto F = lt(size, D);
           auto St = lt(stride, D); Int n = m.getNActive(IS);
           auto I = ft(in, {n, inStride}); auto O = torch::empty({0}, at::kFloat);
           (void)nPlanes;
           cpu_MaxPooling_updateOutput<float, D>(IS, OS, F, St, m, I, O, nFeaturesToDrop);
           copy_out(O, out));
}
void ref_avgpool(void *h, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                 const int64_t *stride, const float *in, int inStride, float *out, int nPlanes,
                 int nFeaturesToDrop) {
  DISPATCH(h, auto IS = lt(inSz, D); auto OS = lt(outSz, D); auto F = lt(size, D);
           auto St = lt(stride, D); Int n = m.getNActive(IS);
           auto I = ft(in, {n, inStride}); auto O = torch::empty({0}, at::kFloat);
           (void)nPlanes;
           cpu_AveragePooling_updateOutput<float, D>(IS, OS, F, St, m, I, O, nFeaturesToDrop);
           copy_out(O, out));
}
void ref_unpool(void *h, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                const int64_t *stride, const float *in, int inStride, float *out, int nPlanes,
                int nFeaturesToDrop) {
  DISPATCH(h, auto IS = lt(inSz, D); auto OS = lt(outSz, D); auto F = lt(size, D);
           auto St = lt(stride, D); Int n = m.getNActive(IS);
           auto I = ft(in, {n, inStride}); auto O = torch::empty({0}, at::kFloat);
           (void)nPlanes;
           cpu_UnPooling_updateOutput<float, D>(IS, OS, F, St, m, I, O, nFeaturesToDrop);
           copy_out(O, out));
}
double ref_nin(const float *in, float *out, const float *w, const float *bias, int nActive, int nIn,
               int nOut) {
  auto I = ft(in, {nActive, nIn});
  auto O = torch::empty({0}, at::kFloat);
  auto W = ft(w, {nIn, nOut});
  auto B = ft(bias, {nOut});
  double macs = cpu_NetworkInNetwork_updateOutput<float>(I, O, W, B);
  copy_out(O, out);
  return macs;
}
void ref_bn_eval(const float *in, float *out, int nActive, int nPlanes, int inStride,
                 int outStride, const float *runningMean, const float *runningVar,
                 const float *weight, const float *bias, float eps, float leakiness) {
  std::vector<float> sm(nPlanes), si(nPlanes);
  BatchNormalization_ForwardPass<float>((float *)in, out, nPlanes, inStride, outStride, nActive,
                                        sm.data(), si.data(), (float *)runningMean,
                                        (float *)runningVar, (float *)weight, (float *)bias, eps,
                                        0.99f, false, leakiness);
}
void ref_input_fwd(void *h, const float *in, float *out, int nPlanes) {
  // The rule list was built by ref_input_layer; this is the body of
  // cpu_InputLayer_updateOutput after m.inputLayer(...) (CPU/IOLayers.cpp:57-71).
  DISPATCH(h, (void)D; auto &rules = m.inputLayerRuleBook; Int mode = rules[0][0];
           Int maxActive = rules[0][1]; Int nRows = rules[0][3];
           if (mode == 0) { std::memcpy(out, in, sizeof(float) * (size_t)rules[0][2] * nPlanes); }
           else {
             std::memset(out, 0, sizeof(float) * (size_t)nRows * nPlanes);
             InputLayer_ForwardPass<float>((float *)in, out, nRows, maxActive, nPlanes,
                                           &rules[1][0], mode == 4);
           });
}
void ref_output_fwd(void *h, const float *in, float *out, int nPlanes) {
  DISPATCH(h, auto I = ft(in, {(int64_t)m.inputLayerRuleBook[0][3], nPlanes});
           auto O = torch::empty({0}, at::kFloat);
           cpu_OutputLayer_updateOutput<float, D>(m, I, O); copy_out(O, out));
}
int ref_bl_input_layer(void *h, const int64_t *spatial, const int64_t *coords, int batchSize,
                       int length, int mode) {
  int r = 0;
  DISPATCH(h, auto S = lt(spatial, D);
           auto C = torch::from_blob((void *)coords, {batchSize, length, D}, at::kLong).clone();
           m.blLayer(S, C, mode); r = *m.inputNActive);
  return r;
}
void ref_bl_rules_header(void *h, int *hdr) {
  DISPATCH(h, (void)D; for (int i = 0; i < 5; i++) hdr[i] = m.blLayerRuleBook[0][i]);
}
void ref_bl_rules(void *h, int *rows) {
  DISPATCH(h, (void)D; if (m.blLayerRuleBook.size() > 1) std::memcpy(
                           rows, m.blLayerRuleBook[1].data(),
                           m.blLayerRuleBook[1].size() * sizeof(Int)));
}
void ref_bl_input_fwd(void *h, const float *in, float *out, int nPlanes) {
  // The rule list was built by ref_bl_input_layer; this is the body of
  // cpu_BLInputLayer_updateOutput after m.blLayer(...) (CPU/IOLayers.cpp:126-138).
  DISPATCH(h, (void)D; auto &rules = m.blLayerRuleBook; Int mode = rules[0][0];
           Int maxActive = rules[0][1]; Int nRows = rules[0][4];
           if (mode == 0) { std::memcpy(out, in, sizeof(float) * (size_t)nRows * nPlanes); }
           else {
             std::memset(out, 0, sizeof(float) * (size_t)nRows * nPlanes);
             InputLayer_ForwardPass<float>((float *)in, out, nRows, maxActive, nPlanes,
                                           &rules[1][0], mode == 4);
           });
}
void ref_bl_output_fwd(void *h, const float *in, float *out, int nPlanes) {
  DISPATCH(h, auto I = ft(in, {(int64_t)m.blLayerRuleBook[0][4], nPlanes});
           auto O = torch::empty({0}, at::kFloat);
           cpu_BLOutputLayer_updateOutput<float, D>(m, I, O); copy_out(O, out));
}
void ref_s2d(void *h, const int64_t *spatial, const float *in, float *out, int nPlanes) {
  DISPATCH(h, auto S = lt(spatial, D); Int n = m.getNActive(S); auto I = ft(in, {n, nPlanes});
           auto O = torch::empty({0}, at::kFloat);
           cpu_SparseToDense_updateOutput<float, D>(S, m, I, O, nPlanes); copy_out(O, out));
}

// sparseconvnet/inputBatch.py's calls into Metadata, with the feature tensor it passes along
// kept in the handle.
void ref_set_input_spatial_size(void *h, const int64_t *spatial) {
  DISPATCH(h, auto S = lt(spatial, D); m.setInputSpatialSize(S));
}
void ref_batch_add_sample(void *h) { DISPATCH(h, (void)D; m.batchAddSample()); }
int ref_set_input_locations(void *h, const int64_t *locations, int n, int ncols, const float *vecs,
                            int nPlanes, int overwrite) {
  int r = 0;
  DISPATCH(h, if (ncols == D && !m.inputSG) { r = -1; break; }
           auto L = torch::from_blob((void *)locations, {n, ncols}, at::kLong).clone();
           auto V = ft(vecs, {n, nPlanes}).clone();
           m.setInputSpatialLocations(((Handle *)h)->feats, L, V, overwrite != 0));
  return r;
}
void ref_add_sample_from_tensor(void *h, const float *tensor, const int64_t *size, int nPlanes,
                                const int64_t *offset, float threshold) {
  DISPATCH(h, std::vector<int64_t> shape(size, size + D); shape.push_back(nPlanes);
           auto T = ft(tensor, shape).clone(); auto O = lt(offset, D);
           auto S = torch::empty({D}, at::kLong);
           for (int i = 0; i < D; i++) S.data_ptr<long>()[i] = m.inputSpatialSize[i];
           m.addSampleFromThresholdedTensor(((Handle *)h)->feats, T, O, S, threshold));
}
int ref_batch_planes(void *h) {
  auto &f = ((Handle *)h)->feats;
  return f.dim() == 2 ? (int)f.size(1) : 0;
}
void ref_batch_features(void *h, float *out) { copy_out(((Handle *)h)->feats, out); }
void ref_generate_rulebooks(void *h, int size) {
  DISPATCH(h, (void)D; if (size == 2) m.generateRuleBooks2s2(); else m.generateRuleBooks3s2());
}

// ---- backward pass: the reference's own functions behind the oracle's signatures --------------

void ref_subm_conv_bwd(void *h, const int64_t *spatial, const int64_t *filter, const float *in, float *d_in,
                       const float *d_out, const float *w, float *d_w, float *d_bias, int nIn, int nOut,
                       int groups) {
  DISPATCH(h, auto S = lt(spatial, D); auto F = lt(filter, D); Int n = m.getNActive(S);
           int64_t K = F.prod().item<int64_t>();
           auto I = ft(in, {n, nIn}); auto DI = torch::empty({0}, at::kFloat);
           auto DO = ft(d_out, {n, nOut}).clone();
           auto W = ft(w, {K, groups, nIn / groups, nOut / groups});
           auto DW = torch::zeros({K, groups, nIn / groups, nOut / groups}, at::kFloat);
           auto DB = d_bias ? torch::zeros({nOut}, at::kFloat) : torch::empty({0}, at::kFloat);
           cpu_SubmanifoldConvolution_backward<float, D>(S, F, m, I, DI, DO, W, DW, DB);
           copy_out(DI, d_in); copy_out(DW, d_w); if (d_bias) copy_out(DB, d_bias));
}
void ref_conv_bwd(void *h, const int64_t *inSz, const int64_t *outSz, const int64_t *filter,
                  const int64_t *stride, const float *in, float *d_in, const float *d_out, const float *w,
                  float *d_w, float *d_bias, int nIn, int nOut, int groups) {
  DISPATCH(h, auto IS = lt(inSz, D); auto OS = lt(outSz, D); auto F = lt(filter, D); auto St = lt(stride, D);
           Int n = m.getNActive(IS); Int no = m.getNActive(OS); int64_t K = F.prod().item<int64_t>();
           auto I = ft(in, {n, nIn}); auto DI = torch::empty({0}, at::kFloat);
           auto DO = ft(d_out, {no, nOut}).clone();
           auto W = ft(w, {K, groups, nIn / groups, nOut / groups});
           auto DW = torch::zeros({K, groups, nIn / groups, nOut / groups}, at::kFloat);
           auto DB = d_bias ? torch::zeros({nOut}, at::kFloat) : torch::empty({0}, at::kFloat);
           cpu_Convolution_backward<float, D>(IS, OS, F, St, m, I, DI, DO, W, DW, DB);
           copy_out(DI, d_in); copy_out(DW, d_w); if (d_bias) copy_out(DB, d_bias));
}
void ref_deconv_bwd(void *h, const int64_t *inSz, const int64_t *outSz, const int64_t *filter,
                    const int64_t *stride, const float *in, float *d_in, const float *d_out, const float *w,
                    float *d_w, float *d_bias, int nIn, int nOut, int groups) {
  DISPATCH(h, auto IS = lt(inSz, D); auto OS = lt(outSz, D); auto F = lt(filter, D); auto St = lt(stride, D);
           Int n = m.getNActive(IS); Int no = m.getNActive(OS); int64_t K = F.prod().item<int64_t>();
           auto I = ft(in, {n, nIn}); auto DI = torch::empty({0}, at::kFloat);
           auto DO = ft(d_out, {no, nOut}).clone();
           auto W = ft(w, {K, groups, nIn / groups, nOut / groups});
           auto DW = torch::zeros({K, groups, nIn / groups, nOut / groups}, at::kFloat);
           auto DB = d_bias ? torch::zeros({nOut}, at::kFloat) : torch::empty({0}, at::kFloat);
           cpu_Deconvolution_backward<float, D>(IS, OS, F, St, m, I, DI, DO, W, DW, DB);
           copy_out(DI, d_in); copy_out(DW, d_w); if (d_bias) copy_out(DB, d_bias));
}
void ref_nin_bwd(const float *in, float *d_in, const float *d_out, const float *w, float *d_w, float *d_bias,
                 int nActive, int nIn, int nOut) {
  auto I = ft(in, {nActive, nIn});
  auto DO = ft(d_out, {nActive, nOut}).clone();
  auto W = ft(w, {nIn, nOut});
  auto DI = torch::empty({0}, at::kFloat);
  auto DW = torch::zeros({nIn, nOut}, at::kFloat);
  auto DB = d_bias ? torch::zeros({nOut}, at::kFloat) : torch::empty({0}, at::kFloat);
  cpu_NetworkInNetwork_updateGradInput<float>(DI, DO, W);
  cpu_NetworkInNetwork_accGradParameters<float>(I, DO, DW, DB);
  copy_out(DI, d_in);
  copy_out(DW, d_w);
  if (d_bias) copy_out(DB, d_bias);
}
void ref_bn_train(const float *in, float *out, int nActive, int nPlanes, int inStride, int outStride,
                  float *saveMean, float *saveInvStd, float *runningMean, float *runningVar,
                  const float *weight, const float *bias, float eps, float momentum, float leakiness) {
  BatchNormalization_ForwardPass<float>((float *)in, out, nPlanes, inStride, outStride, nActive, saveMean,
                                        saveInvStd, runningMean, runningVar, (float *)weight, (float *)bias, eps,
                                        momentum, true, leakiness);
}
void ref_bn_bwd(const float *in, float *d_in, const float *out, const float *d_out, int nActive, int nPlanes,
                int inStride, int outStride, const float *saveMean, const float *saveInvStd,
                const float *weight, float *d_weight, float *d_bias, float leakiness) {
  std::vector<float> d((size_t)nActive * outStride);  // the reference scales d_out in place
  std::memcpy(d.data(), d_out, d.size() * sizeof(float));
  BatchNormalization_BackwardPass<float>((float *)in, d_in, (float *)out, d.data(), nPlanes, inStride, outStride,
                                         nActive, (float *)saveMean, (float *)saveInvStd, nullptr, nullptr,
                                         (float *)weight, nullptr, d_weight, d_bias, leakiness);
}
void ref_maxpool_bwd(void *h, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                     const int64_t *stride, const float *in, float *d_in, int inStride, const float *out,
                     const float *d_out, int nPlanes, int nFeaturesToDrop) {
  DISPATCH(h, auto IS = lt(inSz, D); auto OS = lt(outSz, D); auto F = lt(size, D); auto St = lt(stride, D);
           Int n = m.getNActive(IS); Int no = m.getNActive(OS);
           auto I = ft(in, {n, inStride}); auto DI = torch::empty({0}, at::kFloat);
           auto O = ft(out, {no, nPlanes}); auto DO = ft(d_out, {no, nPlanes});
           cpu_MaxPooling_updateGradInput<float, D>(IS, OS, F, St, m, I, DI, O, DO, nFeaturesToDrop);
           copy_out(DI, d_in));
}
void ref_avgpool_bwd(void *h, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                     const int64_t *stride, float *d_in, int inStride, const float *d_out, int nPlanes,
                     int nFeaturesToDrop) {
  DISPATCH(h, auto IS = lt(inSz, D); auto OS = lt(outSz, D); auto F = lt(size, D); auto St = lt(stride, D);
           Int n = m.getNActive(IS); Int no = m.getNActive(OS);
           auto I = torch::zeros({n, inStride}, at::kFloat); auto DI = torch::empty({0}, at::kFloat);
           auto DO = ft(d_out, {no, nPlanes});
           cpu_AveragePooling_updateGradInput<float, D>(IS, OS, F, St, m, I, DI, DO, nFeaturesToDrop);
           copy_out(DI, d_in));
}
void ref_unpool_bwd(void *h, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                    const int64_t *stride, float *d_in, int inStride, const float *d_out, int nPlanes,
                    int nFeaturesToDrop) {
  DISPATCH(h, auto IS = lt(inSz, D); auto OS = lt(outSz, D); auto F = lt(size, D); auto St = lt(stride, D);
           Int n = m.getNActive(IS); Int no = m.getNActive(OS);
           auto DI = torch::zeros({n, inStride}, at::kFloat);  // sparseconvnet/unPooling.py:49
           auto DO = ft(d_out, {no, nPlanes});
           cpu_UnPooling_updateGradInput<float, D>(IS, OS, F, St, m, DI, DO, nFeaturesToDrop);
           copy_out(DI, d_in));
}
void ref_input_bwd(void *h, float *d_in, const float *d_out, int nPlanes) {
  DISPATCH(h, auto &rules = m.inputLayerRuleBook; Int mode = rules[0][0];
           auto DO = ft(d_out, {(int64_t)(mode == 0 ? rules[0][2] : rules[0][3]), nPlanes});
           auto DI = torch::empty({0}, at::kFloat);
           cpu_InputLayer_updateGradInput<float, D>(m, DI, DO); copy_out(DI, d_in));
}
void ref_output_bwd(void *h, float *d_in, const float *d_out, int nPlanes) {
  DISPATCH(h, auto DO = ft(d_out, {(int64_t)m.inputLayerRuleBook[0][2], nPlanes});
           auto DI = torch::empty({0}, at::kFloat);
           cpu_OutputLayer_updateGradInput<float, D>(m, DI, DO); copy_out(DI, d_in));
}
void ref_bl_input_bwd(void *h, float *d_in, const float *d_out, int nPlanes) {
  DISPATCH(h, auto DO = ft(d_out, {(int64_t)m.blLayerRuleBook[0][4], nPlanes});
           auto DI = torch::empty({0}, at::kFloat);
           cpu_BLInputLayer_updateGradInput<float, D>(m, DI, DO); copy_out(DI, d_in));
}
void ref_bl_output_bwd(void *h, float *d_in, const float *d_out, int nPlanes) {
  DISPATCH(h, auto DO = ft(d_out, {(int64_t)m.blLayerRuleBook[0][2], (int64_t)m.blLayerRuleBook[0][3], nPlanes});
           auto DI = torch::empty({0}, at::kFloat);
           cpu_BLOutputLayer_updateGradInput<float, D>(m, DI, DO); copy_out(DI, d_in));
}
void ref_s2d_bwd(void *h, const int64_t *spatial, float *d_in, const float *d_out, int nPlanes) {
  DISPATCH(h, auto S = lt(spatial, D); Int n = m.getNActive(S);
           auto I = torch::zeros({n, nPlanes}, at::kFloat); auto DI = torch::empty({0}, at::kFloat);
           std::vector<int64_t> shape{(int64_t)m.getBatchSize(S), nPlanes};
           for (int i = 0; i < D; i++) shape.push_back(spatial[i]);
           auto DO = ft(d_out, shape);
           cpu_SparseToDense_updateGradInput<float, D>(S, m, I, DI, DO); copy_out(DI, d_in));
}

// ActivePooling_updateOutput / _updateGradInput (pybind.cpp:34-43).  The reference's rule builder
// (Metadata/ActivePoolingRules.h:29) only returns when no sample holds more than one site; for
// anything else these return 0 without calling it.
static int active_pooling_terminates(void *h, const int64_t *spatial) {
  int ok = 1;
  DISPATCH(h, auto S = lt(spatial, D); auto &SGs = m.getSparseGrid(S); for (auto &sg : SGs) if (sg.mp.size() != 1) ok = 0);
  return ok;
}
int ref_active_pooling(void *h, const int64_t *spatial, const float *in, float *out, int nPlanes, int average) {
  if (!active_pooling_terminates(h, spatial)) return 0;
  DISPATCH(h, auto S = lt(spatial, D); Int n = m.getNActive(S); auto I = ft(in, {n, nPlanes});
           auto O = torch::empty({0}, at::kFloat);
           cpu_ActivePooling_updateOutput<float, D>(S, m, I, O, average != 0); copy_out(O, out));
  return 1;
}
int ref_active_pooling_bwd(void *h, const int64_t *spatial, float *d_in, const float *d_out, int nPlanes, int average) {
  if (!active_pooling_terminates(h, spatial)) return 0;
  DISPATCH(h, auto S = lt(spatial, D); Int n = m.getNActive(S); auto I = torch::zeros({n, nPlanes}, at::kFloat);
           auto DI = torch::empty({0}, at::kFloat);
           auto DO = ft(d_out, {(int64_t)m.getSparseGrid(S).size(), nPlanes});
           cpu_ActivePooling_updateGradInput<float, D>(S, m, I, DI, DO, average != 0); copy_out(DI, d_in));
  return 1;
}
}  // extern "C"
