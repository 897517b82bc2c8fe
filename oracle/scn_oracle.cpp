// CPU oracle for the sparse-convolution path (forward and backward).
//
// TEST INFRASTRUCTURE ONLY.  This file restates, on the CPU, the algorithm of
// the reference implementation (facebookresearch/SparseConvNet, directory
// sparseconvnet/SCN) for the forward pass: coordinate hash grids, rulebook
// generation, gather -> GEMM -> scatter-add convolutions, eval-mode batch
// norm, max pooling and the input / output / sparse-to-dense layers.  It is
// the checker the GPU library is compared with and the "port" flavour of the
// CPU baseline; nothing in the shipped library links or calls it.
//
// Every function cites the reference file:line it follows.  Row numbering of
// levels created by a strided convolution follows this file's own hash-bucket
// iteration, as the reference's follows google::dense_hash_map's; comparisons
// therefore go through coordinates (orc_spatial_locations), never raw rows.
//
// Pinned by tests/test_oracle_*.py: brute-force dictionaries on small inputs,
// dense torch convolutions / pooling / batch-norm, closed-form invariants, and
// (where oracle/_ref builds) the compiled reference itself.
//
// Build: g++ -O3 -fopenmp -shared -fPIC scn_oracle.cpp -o libscn_oracle.so

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <vector>

typedef int32_t Int;  // Metadata/32bits.h:11
static const int MAXD = 6;  // sparseconvnet_cpu.cpp:14-20 instantiates 1..6

struct Pt {
  Int x[MAXD];
};

// Open-addressing map Point -> Int.  Hash function as Metadata/32bits.h:57-66
// (32-bit wrap-around multiply by 2166136261 then xor, seed 16777619).
// Iteration is in bucket order, as with the reference's dense_hash_map
// (Metadata/Metadata.h:24-28); the probe sequence and growth policy are this
// file's own, so the order differs from the reference's, which is allowed.
struct Grid {
  Int ctr = 0;  // Metadata/Metadata.h:31
  int dim = 0;
  std::vector<Pt> keys;
  std::vector<Int> vals;
  std::vector<uint8_t> used;
  size_t count = 0;
  void init(int d) {
    dim = d;
    keys.assign(32, Pt());
    vals.assign(32, 0);
    used.assign(32, 0);
    count = 0;
  }
  size_t hash(const Pt &p) const {
    uint32_t h = 16777619u;
    for (int i = 0; i < dim; i++) {
      h *= 2166136261u;
      h ^= (uint32_t)p.x[i];
    }
    return (size_t)(int64_t)(int32_t)h;
  }
  bool eq(const Pt &a, const Pt &b) const {
    for (int i = 0; i < dim; i++)
      if (a.x[i] != b.x[i]) return false;
    return true;
  }
  void grow() {
    std::vector<Pt> ok;
    std::vector<Int> ov;
    std::vector<uint8_t> ou;
    ok.swap(keys);
    ov.swap(vals);
    ou.swap(used);
    size_t nb = ou.size() * 2;
    keys.assign(nb, Pt());
    vals.assign(nb, 0);
    used.assign(nb, 0);
    count = 0;
    for (size_t i = 0; i < ou.size(); i++)
      if (ou[i]) *insert(ok[i], ov[i]).first = ov[i];
  }
  // Returns (pointer to value, inserted?) like dense_hash_map::insert.
  std::pair<Int *, bool> insert(const Pt &p, Int v) {
    if ((count + 1) * 2 > used.size()) grow();
    size_t mask = used.size() - 1, b = hash(p) & mask;
    while (used[b]) {
      if (eq(keys[b], p)) return {&vals[b], false};
      b = (b + 1) & mask;
    }
    used[b] = 1;
    keys[b] = p;
    vals[b] = v;
    count++;
    return {&vals[b], true};
  }
  const Int *find(const Pt &p) const {
    size_t mask = used.size() - 1, b = hash(p) & mask;
    while (used[b]) {
      if (eq(keys[b], p)) return &vals[b];
      b = (b + 1) & mask;
    }
    return nullptr;
  }
};

typedef std::vector<Grid> Grids;                 // Metadata/Metadata.h:34
typedef std::vector<std::vector<Int>> RuleBook;  // Metadata/Metadata.h:35
typedef std::vector<int64_t> Key;

// Metadata/Metadata.h:44-74: per-spatial-size active counts and grids, and
// lazily built rulebooks cached by (size || filter [|| stride]).
struct Metadata {
  int dim;
  std::map<Key, Int> nActive;
  std::map<Key, Grids> grids;
  RuleBook inputLayerRuleBook;
  RuleBook blLayerRuleBook;
  std::map<Key, RuleBook> submanifoldRuleBooks;
  std::map<Key, RuleBook> ruleBooks;
  std::map<Key, RuleBook> sparseToDenseRuleBooks;
  Key inputSpatialSize;
  // point-at-a-time input (Metadata/Metadata.h:62-64 inputSGs / inputSG / inputNActive, and
  // the feature tensor that sparseconvnet/inputBatch.py:18 hands to every call)
  Int currentSample = -1;
  int batchPlanes = 0;
  std::vector<float> batchFeatures;
};

static Key mkkey(int dim, const int64_t *a, const int64_t *b = nullptr,
                 const int64_t *c = nullptr) {
  Key k(a, a + dim);
  if (b) k.insert(k.end(), b, b + dim);
  if (c) k.insert(k.end(), c, c + dim);
  return k;
}

static void resize_grids(Grids &g, size_t n, int dim) {
  size_t old = g.size();
  g.resize(n);
  for (size_t i = old; i < n; i++) g[i].init(dim);
}

static Int volume(int dim, const int64_t *s) {  // Metadata/Metadata.cpp volume<>
  Int v = 1;
  for (int i = 0; i < dim; i++) v *= (Int)s[i];
  return v;
}

// Metadata/IOLayersRules.h:18-121
static void inputLayerRules(Grids &SGs, RuleBook &rules, const int64_t *coords,
                            Int nInputRows, Int nInputColumns, Int batchSize,
                            Int mode, Int &nActive, int dim) {
  resize_grids(SGs, batchSize, dim);  // :25 minimum batch size
  Pt p = Pt();
  if (mode == 0) {  // :28-58
    nActive = nInputRows;
    rules.resize(1);
    rules[0] = {mode, 1, nInputRows, nInputRows};
    if (nInputColumns == dim) {
      SGs.clear();
      resize_grids(SGs, 1, dim);
      for (Int i = 0; i < nInputRows; ++i) {
        for (int j = 0; j < dim; j++) p.x[j] = (Int)coords[j];
        coords += dim;
        *SGs[0].insert(p, i).first = i;
      }
    } else {
      for (Int i = 0; i < nInputRows; ++i) {
        for (int j = 0; j < dim; j++) p.x[j] = (Int)coords[j];
        Int idx = (Int)coords[dim];
        coords += dim + 1;
        if (idx + 1 >= (Int)SGs.size()) resize_grids(SGs, idx + 1, dim);
        *SGs[idx].insert(p, i).first = i;
      }
    }
    return;
  }
  std::vector<std::vector<Int>> outputRows;  // :61-89
  if (nInputColumns == dim) {
    SGs.clear();
    resize_grids(SGs, 1, dim);
  }
  for (Int i = 0; i < nInputRows; ++i) {
    for (int j = 0; j < dim; j++) p.x[j] = (Int)coords[j];
    Int idx = 0;
    if (nInputColumns == dim) {
      coords += dim;
    } else {
      idx = (Int)coords[dim];
      coords += dim + 1;
      if (idx + 1 >= (Int)SGs.size()) resize_grids(SGs, idx + 1, dim);
    }
    auto r = SGs[idx].insert(p, nActive);
    if (r.second) outputRows.resize(++nActive);
    outputRows[*r.first].push_back(i);
  }
  rules.resize(2);  // :90-94
  rules[0] = {mode, 1, nInputRows, (Int)outputRows.size()};
  auto &rule = rules[1];
  if (mode == 1)  // :96-101 first occurrence
    for (Int i = 0; i < nActive; ++i) {
      rule.push_back(1);
      rule.push_back(outputRows[i].front());
    }
  if (mode == 2)  // :102-107 last occurrence
    for (Int i = 0; i < nActive; ++i) {
      rule.push_back(1);
      rule.push_back(outputRows[i].back());
    }
  if (mode == 3 || mode == 4) {  // :108-119
    Int maxActive = 0;
    for (auto &row : outputRows) maxActive = std::max(maxActive, (Int)row.size());
    rules[0][1] = maxActive;
    for (auto &row : outputRows) {
      rule.push_back((Int)row.size());
      for (auto r : row) rule.push_back(r);
      rule.resize((rule.size() + maxActive) / (maxActive + 1) * (maxActive + 1));
    }
  }
}

// Metadata/IOLayersRules.h:132-286.  coords is [batchSize, length, dim]; a position whose
// first coordinate is negative is empty.  Header (:122-128):
// [mode, maxActive, batchSize, length, nOutputRows]; rows nOutputRows x (1 + maxActive).
// Mode 1 keeps the LAST point of a site (:184-190), mode 2 the first (:199-207).
static void blRules(Grids &SGs, RuleBook &rules, const int64_t *coords, Int batchSize, Int length,
                    Int mode, Int &nActive, int dim) {
  SGs.clear();
  resize_grids(SGs, batchSize, dim);
  Pt p = Pt();
  if (mode == 0) {  // :141-162 every position is its own row
    nActive = batchSize * length;
    rules.resize(1);
    rules[0] = {mode, 1, batchSize, length, nActive};
    for (Int I = 0; I < batchSize; I++) {
      SGs[I].ctr = I * length;
      const int64_t *c = coords + (size_t)I * length * dim;
      for (Int l = 0; l < length; ++l, c += dim) {
        for (int j = 0; j < dim; j++) p.x[j] = (Int)c[j];
        *SGs[I].insert(p, l).first = l;
      }
    }
    return;
  }
  // per sample: the input rows of every output row, in input order (:165-252)
  std::vector<std::vector<std::vector<Int>>> outputRows(batchSize);
  for (Int I = 0; I < batchSize; I++) {
    auto &ors = outputRows[I];
    const int64_t *c = coords + (size_t)I * length * dim;
    Int i = I * length;
    for (Int l = 0; l < length; ++l, ++i, c += dim) {
      for (int j = 0; j < dim; j++) p.x[j] = (Int)c[j];
      if (p.x[0] < 0) continue;
      auto r = SGs[I].insert(p, (Int)ors.size());
      if (r.second) ors.emplace_back();
      ors[*r.first].push_back(i);
    }
  }
  for (Int I = 0; I < batchSize; I++) {  // :209-212,254-257
    SGs[I].ctr = nActive;
    nActive += (Int)outputRows[I].size();
  }
  Int maxActive = 1;
  if (mode >= 3)
    for (auto &ors : outputRows)
      for (auto &row : ors) maxActive = std::max(maxActive, (Int)row.size());
  rules.resize(2);
  rules[0] = {mode, maxActive, batchSize, length, nActive};
  auto &rule = rules[1];
  rule.assign((size_t)(maxActive + 1) * nActive, 0);
  for (Int I = 0; I < batchSize; I++) {
    Int *rr = rule.data() + (size_t)SGs[I].ctr * (maxActive + 1);
    for (auto &row : outputRows[I]) {
      if (mode == 1) {
        rr[0] = 1, rr[1] = row.back();
      } else if (mode == 2) {
        rr[0] = 1, rr[1] = row.front();
      } else {
        rr[0] = (Int)row.size();
        for (size_t q = 0; q < row.size(); q++) rr[1 + q] = row[q];
      }
      rr += 1 + maxActive;
    }
  }
}

// Row-major offset of p inside the box [lb, ub], last dimension fastest:
// Metadata/RectangularRegions.h:30-38.
static Int region_offset(int dim, const Int *lb, const Int *ub, const Int *p) {
  Int of = 0, m = 1;
  for (int i = dim - 1; i >= 0; i--) {
    of += m * (p[i] - lb[i]);
    m *= ub[i] - lb[i] + 1;
  }
  return of;
}

// Visit every point of the box [lb, ub] with the last dimension fastest
// (Metadata/RectangularRegions.h:43-71).  Empty when some lb[i] > ub[i].
template <class F>
static void for_region(int dim, const Int *lb, const Int *ub, F f) {
  Pt p = Pt();
  for (int i = 0; i < dim; i++) {
    if (lb[i] > ub[i]) return;
    p.x[i] = lb[i];
  }
  for (;;) {
    f(p);
    int i = dim - 1;
    for (;;) {
      if (++p.x[i] <= ub[i]) break;
      p.x[i] = lb[i];
      if (--i < 0) return;
    }
  }
}

// Metadata/SubmanifoldConvolutionRules.h:11-45
static double subm_SgToRules(const Grid &grid, RuleBook &rules,
                             const int64_t *size, int dim) {
  double count = 0;
  for (size_t b = 0; b < grid.used.size(); b++) {
    if (!grid.used[b]) continue;
    const Pt &out = grid.keys[b];
    Int lb[MAXD], ub[MAXD];
    for (int i = 0; i < dim; i++) {
      Int pad = (Int)size[i] / 2;
      lb[i] = out.x[i] - pad;
      ub[i] = out.x[i] + (Int)size[i] - 1 - pad;
    }
    Int rulesOffset = 0;
    for_region(dim, lb, ub, [&](const Pt &in) {
      const Int *v = grid.find(in);
      if (v) {
        rules[rulesOffset].push_back(*v + grid.ctr);
        rules[rulesOffset].push_back(grid.vals[b] + grid.ctr);
        count++;
      }
      rulesOffset++;
    });
  }
  return count;
}

// Metadata/SubmanifoldConvolutionRules.h:59-87: samples in parallel, then
// per-offset concatenation in sample order.
static void subm_SgsToRules(const Grids &SGs, RuleBook &rules,
                            const int64_t *size, int dim) {
  Int sd = volume(dim, size);
  std::vector<RuleBook> rbs(SGs.size());
  rules.clear();
  rules.resize(sd);
#pragma omp parallel for schedule(dynamic, 1)
  for (Int i = 0; i < (Int)SGs.size(); i++) {
    rbs[i].resize(sd);
    subm_SgToRules(SGs[i], rbs[i], size, dim);
  }
#pragma omp parallel for
  for (Int k = 0; k < sd; k++)
    for (auto &rb : rbs) rules[k].insert(rules[k].end(), rb[k].begin(), rb[k].end());
}

// Metadata/ConvolutionRules.h:11-34 with the region calculators of
// Metadata/RectangularRegions.h:95-119.
static void conv_InputSgToRulesAndOutputSg(const Grid &inG, Grid &outG,
                                           RuleBook &rules, const int64_t *size,
                                           const int64_t *stride,
                                           const int64_t *outSz, int dim) {
  rules.resize(volume(dim, size));
  for (size_t b = 0; b < inG.used.size(); b++) {
    if (!inG.used[b]) continue;
    const Pt &in = inG.keys[b];
    Int lb[MAXD], ub[MAXD];
    for (int i = 0; i < dim; i++) {  // OutputRegionCalculator :109-119
      lb[i] = (Int)std::max<int64_t>(0, (in.x[i] - size[i] + stride[i]) / stride[i]);
      ub[i] = (Int)std::min<int64_t>(outSz[i] - 1, in.x[i] / stride[i]);
    }
    for_region(dim, lb, ub, [&](const Pt &j) {
      Int ilb[MAXD], iub[MAXD];
      for (int i = 0; i < dim; i++) {  // InputRegionCalculator :95-105
        ilb[i] = j.x[i] * (Int)stride[i];
        iub[i] = ilb[i] + (Int)size[i] - 1;
      }
      Int rulesOffset = region_offset(dim, ilb, iub, in.x);
      auto mv = outG.insert(j, 0);
      if (mv.second) *mv.first = outG.ctr++;
      rules[rulesOffset].push_back(inG.vals[b] + inG.ctr);
      rules[rulesOffset].push_back(*mv.first);
    });
  }
}

// Metadata/ConvolutionRules.h:61-105
static Int conv_InputSgsToRulesAndOutputSgs(const Grids &inSGs, Grids &outSGs,
                                            RuleBook &rules, const int64_t *size,
                                            const int64_t *stride,
                                            const int64_t *outSz, int dim) {
  rules.clear();
  rules.resize(volume(dim, size));
  outSGs.clear();
  Int batchSize = (Int)inSGs.size();
  resize_grids(outSGs, batchSize, dim);
  std::vector<RuleBook> rbs(batchSize);
#pragma omp parallel for schedule(dynamic, 1)
  for (Int i = 0; i < batchSize; i++)
    conv_InputSgToRulesAndOutputSg(inSGs[i], outSGs[i], rbs[i], size, stride, outSz, dim);
  Int output_nActive = 0;
  for (Int i = 0; i < batchSize; i++) {  // :80-88 ctr <- prefix sum
    Int tmp = output_nActive;
    output_nActive += outSGs[i].ctr;
    outSGs[i].ctr = tmp;
  }
#pragma omp parallel for
  for (Int k = 0; k < (Int)rules.size(); k++) {
    auto &R = rules[k];
    for (Int j = 0; j < batchSize; j++) {
      auto &r = rbs[j][k];
      Int offset = outSGs[j].ctr;
      for (size_t q = 0; q < r.size(); q += 2) {
        R.push_back(r[q]);
        R.push_back(r[q + 1] + offset);
      }
    }
  }
  return output_nActive;
}

// Metadata/ConvolutionRules.h:130-151
static void s2d_rules(const Grids &SGs, RuleBook &rules, const int64_t *spatial, int dim) {
  rules.clear();
  rules.resize(SGs.size());
  Int lb[MAXD], ub[MAXD];
  for (int i = 0; i < dim; i++) {
    lb[i] = 0;
    ub[i] = (Int)spatial[i] - 1;
  }
  for (size_t s = 0; s < SGs.size(); s++) {
    const Grid &g = SGs[s];
    for (size_t b = 0; b < g.used.size(); b++)
      if (g.used[b]) {
        rules[s].push_back(g.vals[b] + g.ctr);
        rules[s].push_back(region_offset(dim, lb, ub, g.keys[b].x));
      }
  }
}

// Metadata/Metadata.cpp:437-451
static RuleBook &getSubmanifoldRuleBook(Metadata &m, const int64_t *spatial, const int64_t *size) {
  auto &rb = m.submanifoldRuleBooks[mkkey(m.dim, spatial, size)];
  if (rb.empty()) subm_SgsToRules(m.grids[mkkey(m.dim, spatial)], rb, size, m.dim);
  return rb;
}
// Metadata/Metadata.cpp:492-518
static RuleBook &getRuleBook(Metadata &m, const int64_t *inSz, const int64_t *outSz,
                             const int64_t *size, const int64_t *stride) {
  auto &rb = m.ruleBooks[mkkey(m.dim, inSz, size, stride)];
  if (rb.empty()) {
    auto &iSGs = m.grids[mkkey(m.dim, inSz)];
    auto &oSGs = m.grids[mkkey(m.dim, outSz)];
    m.nActive[mkkey(m.dim, outSz)] =
        conv_InputSgsToRulesAndOutputSgs(iSGs, oSGs, rb, size, stride, outSz, m.dim);
  }
  return rb;
}
// Metadata/Metadata.cpp:476-491
static RuleBook &getSparseToDenseRuleBook(Metadata &m, const int64_t *spatial) {
  Key k = mkkey(m.dim, spatial);
  auto &SGs = m.grids[k];
  auto &rb = m.sparseToDenseRuleBooks[k];
  if (rb.empty()) s2d_rules(SGs, rb, spatial, m.dim);
  return rb;
}

// C = A[nRules x ip] * W[ip x op], row-major.  Stands in for at::matmul
// (CPU/Convolution.cpp:74,145), a BLAS sgemm that is not part of the
// reference's sources; plain triple loop, fp32 accumulate in k order.
static void sgemm(const float *A, const float *W, float *C, Int n, Int ip, Int op) {
#pragma omp parallel for
  for (Int i = 0; i < n; i++) {
    float *c = C + (size_t)i * op;
    for (Int o = 0; o < op; o++) c[o] = 0.f;
    const float *a = A + (size_t)i * ip;
    for (Int k = 0; k < ip; k++) {
      float av = a[k];
      const float *w = W + (size_t)k * op;
      for (Int o = 0; o < op; o++) c[o] += av * w[o];
    }
  }
}

// The loop shared by CPU/Convolution.cpp:45-79 (strided), :117-150
// (submanifold) and CPU/Deconvolution.cpp:7-41 (columns swapped):
// rule_index_select (:8-24) -> matmul -> rule_index_add_ (:28-43).
static double conv_loop(const RuleBook &rules, int inCol, int outCol, const float *in,
                        float *out, Int nOutRows, const float *w, const float *bias,
                        Int nIn, Int nOut, Int groups) {
  Int ip = nIn / groups, op = nOut / groups;
  for (Int r = 0; r < nOutRows; r++)  // Convolution.cpp:127-131
    for (Int c = 0; c < nOut; c++) out[(size_t)r * nOut + c] = (bias && nOutRows) ? bias[c] : 0.f;
  double flops = 0;
  std::vector<float> A, C;
  for (size_t k = 0; k < rules.size(); k++) {
    const auto &r = rules[k];
    Int nRules = (Int)(r.size() / 2);
    if (!nRules) continue;
    flops += (double)nRules * ip * op * groups;  // Convolution.cpp:141
    A.resize((size_t)nRules * ip);
    C.resize((size_t)nRules * op);
    for (Int g = 0; g < groups; g++) {
      // weight[k][g] is [ip x op] (submanifoldConvolution.py:24-26)
      const float *wk = w + (((size_t)k * groups + g) * ip) * op;
#pragma omp parallel for
      for (Int i = 0; i < nRules; i++)
        std::memcpy(&A[(size_t)i * ip], in + ((size_t)r[2 * i + inCol] * groups + g) * ip,
                    sizeof(float) * ip);
      sgemm(A.data(), wk, C.data(), nRules, ip, op);
#pragma omp parallel for
      for (Int i = 0; i < nRules; i++) {
        float *t = out + ((size_t)r[2 * i + outCol] * groups + g) * op;
        const float *s = &C[(size_t)i * op];
        for (Int j = 0; j < op; j++) t[j] += s[j];
      }
    }
  }
  return flops;
}

extern "C" {

void *orc_md_create(int dim) {
  if (dim < 1 || dim > MAXD) return nullptr;
  Metadata *m = new Metadata();
  m->dim = dim;
  return m;
}
void orc_md_destroy(void *md) { delete (Metadata *)md; }

// Metadata/Metadata.cpp:413-425.  Returns the number of active sites.
int orc_input_layer(void *md, const int64_t *spatial, const int64_t *coords, int n,
                    int ncols, int batchSize, int mode) {
  Metadata &m = *(Metadata *)md;
  m.inputSpatialSize = mkkey(m.dim, spatial);
  Int &nA = m.nActive[m.inputSpatialSize];
  inputLayerRules(m.grids[m.inputSpatialSize], m.inputLayerRuleBook, coords, n, ncols,
                  batchSize, mode, nA, m.dim);
  return nA;
}
// header: [mode, maxActive, nInputRows, nOutputRows]; Metadata/IOLayersRules.h:10-15
void orc_input_rules_header(void *md, int *hdr) {
  Metadata &m = *(Metadata *)md;
  for (int i = 0; i < 4; i++) hdr[i] = m.inputLayerRuleBook[0][i];
}
// rows: nOutputRows x (1 + maxActive); only for mode != 0.
void orc_input_rules(void *md, int *rows) {
  Metadata &m = *(Metadata *)md;
  if (m.inputLayerRuleBook.size() > 1)
    std::memcpy(rows, m.inputLayerRuleBook[1].data(), m.inputLayerRuleBook[1].size() * sizeof(Int));
}
int orc_nactive(void *md, const int64_t *spatial) {  // Metadata/Metadata.cpp:67-70
  Metadata &m = *(Metadata *)md;
  return m.nActive[mkkey(m.dim, spatial)];
}
int orc_batch_size(void *md, const int64_t *spatial) {  // Metadata/Metadata.cpp:171-176
  Metadata &m = *(Metadata *)md;
  return (int)m.grids[mkkey(m.dim, spatial)].size();
}
// Metadata/Metadata.cpp:149-170: out is [nActive, dim+1] int64, zero-filled first.
void orc_spatial_locations(void *md, const int64_t *spatial, int64_t *out) {
  Metadata &m = *(Metadata *)md;
  Key k = mkkey(m.dim, spatial);
  Int nA = m.nActive[k];
  std::memset(out, 0, sizeof(int64_t) * (size_t)nA * (m.dim + 1));
  Grids &SGs = m.grids[k];
  for (size_t s = 0; s < SGs.size(); s++) {
    Grid &g = SGs[s];
    for (size_t b = 0; b < g.used.size(); b++)
      if (g.used[b]) {
        int64_t *o = out + (size_t)(g.vals[b] + g.ctr) * (m.dim + 1);
        for (int d = 0; d < m.dim; d++) o[d] = g.keys[b].x[d];
        o[m.dim] = (int64_t)s;
      }
  }
}

// Rulebook access: kind 0 = submanifold(spatial=a, filter=b),
// 1 = strided(in=a, out=b, filter=c, stride=d), 2 = sparse-to-dense(spatial=a).
// Builds (and caches) on first use, like the getters in Metadata.cpp.
static RuleBook &rb_get(Metadata &m, int kind, const int64_t *a, const int64_t *b,
                        const int64_t *c, const int64_t *d) {
  if (kind == 0) return getSubmanifoldRuleBook(m, a, b);
  if (kind == 1) return getRuleBook(m, a, b, c, d);
  return getSparseToDenseRuleBook(m, a);
}
int orc_rb_noffsets(void *md, int kind, const int64_t *a, const int64_t *b,
                    const int64_t *c, const int64_t *d) {
  return (int)rb_get(*(Metadata *)md, kind, a, b, c, d).size();
}
// counts[k] = number of (first, second) pairs in list k.
void orc_rb_counts(void *md, int kind, const int64_t *a, const int64_t *b, const int64_t *c,
                   const int64_t *d, int64_t *counts) {
  RuleBook &rb = rb_get(*(Metadata *)md, kind, a, b, c, d);
  for (size_t k = 0; k < rb.size(); k++) counts[k] = (int64_t)rb[k].size() / 2;
}
void orc_rb_copy(void *md, int kind, const int64_t *a, const int64_t *b, const int64_t *c,
                 const int64_t *d, int k, int *pairs) {
  RuleBook &rb = rb_get(*(Metadata *)md, kind, a, b, c, d);
  std::memcpy(pairs, rb[k].data(), rb[k].size() * sizeof(Int));
}

// CPU/Convolution.cpp:117-150.  out is [nActive(spatial), nOut]; returns MACs.
double orc_subm_conv(void *md, const int64_t *spatial, const int64_t *filter, const float *in,
                     float *out, const float *w, const float *bias, int nIn, int nOut, int groups) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getSubmanifoldRuleBook(m, spatial, filter);
  return conv_loop(rb, 0, 1, in, out, m.nActive[mkkey(m.dim, spatial)], w, bias, nIn, nOut, groups);
}
// CPU/Convolution.cpp:45-79.  out is [nActive(outSz), nOut].
double orc_conv(void *md, const int64_t *inSz, const int64_t *outSz, const int64_t *filter,
                const int64_t *stride, const float *in, float *out, const float *w,
                const float *bias, int nIn, int nOut, int groups) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getRuleBook(m, inSz, outSz, filter, stride);
  return conv_loop(rb, 0, 1, in, out, m.nActive[mkkey(m.dim, outSz)], w, bias, nIn, nOut, groups);
}
// CPU/Deconvolution.cpp:7-41: rulebook of (outSz -> inSz), gather column 1,
// scatter column 0.  out is [nActive(outSz), nOut].
double orc_deconv(void *md, const int64_t *inSz, const int64_t *outSz, const int64_t *filter,
                  const int64_t *stride, const float *in, float *out, const float *w,
                  const float *bias, int nIn, int nOut, int groups) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getRuleBook(m, outSz, inSz, filter, stride);
  return conv_loop(rb, 1, 0, in, out, m.nActive[mkkey(m.dim, outSz)], w, bias, nIn, nOut, groups);
}
// CPU/MaxPooling.cpp:7-20,37-60.  in is [nIn rows, inStride]; out is
// [nActive(outSz), nPlanes] with nPlanes = C - nFeaturesToDrop, zero-filled first.
void orc_maxpool(void *md, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                 const int64_t *stride, const float *in, int inStride, float *out, int nPlanes,
                 int nFeaturesToDrop) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getRuleBook(m, inSz, outSz, size, stride);
  Int nA = m.nActive[mkkey(m.dim, outSz)];
  std::memset(out, 0, sizeof(float) * (size_t)nA * nPlanes);
  const float *iF = in + nFeaturesToDrop;
  for (auto &r : rb) {
    Int nHot = (Int)(r.size() / 2);
#pragma omp parallel for
    for (Int s = 0; s < nHot; s++) {
      const float *i = iF + (size_t)r[2 * s] * inStride;
      float *o = out + (size_t)r[2 * s + 1] * nPlanes;
      for (Int p = 0; p < nPlanes; p++)
        if (o[p] < i[p]) o[p] = i[p];
    }
  }
}
// CPU/AveragePooling.cpp:7-20,38-61: out zero-filled, then per rule
// out[o] += in[i] / filterVolume with filterVolume = number of rule lists.
void orc_avgpool(void *md, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                 const int64_t *stride, const float *in, int inStride, float *out, int nPlanes,
                 int nFeaturesToDrop) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getRuleBook(m, inSz, outSz, size, stride);
  Int nA = m.nActive[mkkey(m.dim, outSz)];
  std::memset(out, 0, sizeof(float) * (size_t)nA * nPlanes);
  const float *iF = in + nFeaturesToDrop;
  const Int filterVolume = (Int)rb.size();
  for (auto &r : rb) {
    Int nHot = (Int)(r.size() / 2);
    for (Int s = 0; s < nHot; s++) {
      const float *i = iF + (size_t)r[2 * s] * inStride;
      float *o = out + (size_t)r[2 * s + 1] * nPlanes;
      for (Int p = 0; p < nPlanes; p++) o[p] += i[p] / filterVolume;
    }
  }
}
// CPU/UnPooling.cpp:7-20,34-57: the rulebook of (outSz -> inSz), i.e. outSz is the
// finer level; out zero-filled, then out[rule[0]] += in[rule[1]].
void orc_unpool(void *md, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                const int64_t *stride, const float *in, int inStride, float *out, int nPlanes,
                int nFeaturesToDrop) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getRuleBook(m, outSz, inSz, size, stride);
  Int nA = m.nActive[mkkey(m.dim, outSz)];
  std::memset(out, 0, sizeof(float) * (size_t)nA * nPlanes);
  const float *iF = in + nFeaturesToDrop;
  for (auto &r : rb) {
    Int nHot = (Int)(r.size() / 2);
    for (Int s = 0; s < nHot; s++) {
      const float *i = iF + (size_t)r[2 * s + 1] * inStride;
      float *o = out + (size_t)r[2 * s] * nPlanes;
      for (Int p = 0; p < nPlanes; p++) o[p] += i[p];
    }
  }
}
// CPU/NetworkInNetwork.cpp:7-23: out = bias (or 0), then out += in * weight
// (weight [nIn, nOut] row-major); returns nActive * nIn * nOut.
double orc_nin(const float *in, float *out, const float *weight, const float *bias, int nActive,
               int nIn, int nOut) {
#pragma omp parallel for
  for (int row = 0; row < nActive; row++) {
    float *o = out + (size_t)row * nOut;
    for (int q = 0; q < nOut; q++) o[q] = bias ? bias[q] : 0.f;
    const float *i = in + (size_t)row * nIn;
    for (int p = 0; p < nIn; p++) {
      const float v = i[p];
      const float *w = weight + (size_t)p * nOut;
      for (int q = 0; q < nOut; q++) o[q] += v * w[q];
    }
  }
  return (double)nActive * nIn * nOut;
}
// CPU/BatchNormalization.cpp:41-61 (eval branch) and :109-130.
void orc_bn_eval(const float *in, float *out, int nActive, int nPlanes, int inStride,
                 int outStride, const float *runningMean, const float *runningVar,
                 const float *weight, const float *bias, float eps, float leakiness) {
  std::vector<float> w(nPlanes), b(nPlanes);
  for (int p = 0; p < nPlanes; p++) {
    float invStd = powf(runningVar[p] + eps, -0.5f);
    w[p] = invStd * (weight ? weight[p] : 1.f);
    b[p] = -runningMean[p] * w[p] + (bias ? bias[p] : 0.f);
  }
  for (int row = 0; row < nActive; row++) {
    const float *i = in + (size_t)row * inStride;
    float *o = out + (size_t)row * outStride;
    for (int p = 0; p < nPlanes; p++) {
      float v = i[p] * w[p] + b[p];
      const float r = (v > 0) ? 1.f : leakiness;
      o[p] = v * r;
    }
  }
}
// CPU/IOLayers.cpp:11-29,49-72.  out is [nActive, nPlanes].
// CPU/IOLayers.cpp:11-29: out (zero-filled by the caller) += mult * in over each row's list.
static void input_forward_pass(const float *in, float *out, Int nRows, Int maxActive, int nPlanes,
                               const Int *R, bool average) {
#pragma omp parallel for
  for (Int row = 0; row < nRows; row++) {
    const Int *r = R + (size_t)row * (1 + maxActive);
    Int nA = r[0];
    float mult = (average && nA > 0) ? 1.f / nA : 1.f;
    float *o = out + (size_t)row * nPlanes;
    for (Int i = 1; i <= nA; ++i) {
      const float *f = in + (size_t)r[i] * nPlanes;
      for (Int p = 0; p < nPlanes; p++) o[p] += mult * f[p];
    }
  }
}
// CPU/IOLayers.cpp:31-47 with average = false: every listed input point receives its row.
static void input_backward_pass(float *points, const float *rows, Int nRows, Int maxActive, int nPlanes,
                                const Int *R) {
  for (Int row = 0; row < nRows; row++) {
    const Int *r = R + (size_t)row * (1 + maxActive);
    const float *f = rows + (size_t)row * nPlanes;
    for (Int i = 1; i <= r[0]; ++i) {
      float *o = points + (size_t)r[i] * nPlanes;
      for (Int p = 0; p < nPlanes; p++) o[p] += f[p];
    }
  }
}
void orc_input_fwd(void *md, const float *in, float *out, int nPlanes) {
  Metadata &m = *(Metadata *)md;
  auto &rules = m.inputLayerRuleBook;
  Int mode = rules[0][0], maxActive = rules[0][1], nRows = rules[0][3];
  if (mode == 0) {
    std::memcpy(out, in, sizeof(float) * (size_t)rules[0][2] * nPlanes);
    return;
  }
  std::memset(out, 0, sizeof(float) * (size_t)nRows * nPlanes);
  input_forward_pass(in, out, nRows, maxActive, nPlanes, rules[1].data(), mode == 4);
}
// CPU/IOLayers.cpp:95-115 (InputLayer_BackwardPass :31-47 with average=false).
// out is [nInputRows, nPlanes].
void orc_output_fwd(void *md, const float *in, float *out, int nPlanes) {
  Metadata &m = *(Metadata *)md;
  auto &rules = m.inputLayerRuleBook;
  Int mode = rules[0][0], maxActive = rules[0][1], nRows = rules[0][3];
  if (mode == 0) {
    std::memcpy(out, in, sizeof(float) * (size_t)rules[0][2] * nPlanes);
    return;
  }
  std::memset(out, 0, sizeof(float) * (size_t)rules[0][2] * nPlanes);
  input_backward_pass(out, in, nRows, maxActive, nPlanes, rules[1].data());
}
// Metadata/Metadata.cpp:426-436.  Returns the number of active sites.
int orc_bl_input_layer(void *md, const int64_t *spatial, const int64_t *coords, int batchSize,
                       int length, int mode) {
  Metadata &m = *(Metadata *)md;
  m.inputSpatialSize = mkkey(m.dim, spatial);
  Int &nA = m.nActive[m.inputSpatialSize];
  blRules(m.grids[m.inputSpatialSize], m.blLayerRuleBook, coords, batchSize, length, mode, nA, m.dim);
  return nA;
}
void orc_bl_rules_header(void *md, int *hdr) {
  Metadata &m = *(Metadata *)md;
  for (int i = 0; i < 5; i++) hdr[i] = m.blLayerRuleBook[0][i];
}
void orc_bl_rules(void *md, int *rows) {
  Metadata &m = *(Metadata *)md;
  if (m.blLayerRuleBook.size() > 1)
    std::memcpy(rows, m.blLayerRuleBook[1].data(), m.blLayerRuleBook[1].size() * sizeof(Int));
}
// CPU/IOLayers.cpp:117-139.  in is [batchSize * length, nPlanes], out [nActive, nPlanes].
void orc_bl_input_fwd(void *md, const float *in, float *out, int nPlanes) {
  Metadata &m = *(Metadata *)md;
  auto &rules = m.blLayerRuleBook;
  Int mode = rules[0][0], maxActive = rules[0][1], nRows = rules[0][4];
  if (mode == 0) {
    std::memcpy(out, in, sizeof(float) * (size_t)nRows * nPlanes);
    return;
  }
  std::memset(out, 0, sizeof(float) * (size_t)nRows * nPlanes);
  input_forward_pass(in, out, nRows, maxActive, nPlanes, rules[1].data(), mode == 4);
}
// CPU/IOLayers.cpp:186-206.  out is [batchSize * length, nPlanes].
void orc_bl_output_fwd(void *md, const float *in, float *out, int nPlanes) {
  Metadata &m = *(Metadata *)md;
  auto &rules = m.blLayerRuleBook;
  Int mode = rules[0][0], maxActive = rules[0][1], nRows = rules[0][4];
  size_t nPoints = (size_t)rules[0][2] * rules[0][3];
  if (mode == 0) {
    std::memcpy(out, in, sizeof(float) * nPoints * nPlanes);
    return;
  }
  std::memset(out, 0, sizeof(float) * nPoints * nPlanes);
  input_backward_pass(out, in, nRows, maxActive, nPlanes, rules[1].data());
}
// CPU/SparseToDense.cpp:7-19,35-64.  out is [batch, nPlanes, spatial...], zeroed here.
void orc_s2d(void *md, const int64_t *spatial, const float *in, float *out, int nPlanes) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getSparseToDenseRuleBook(m, spatial);
  int64_t vol = 1;
  for (int i = 0; i < m.dim; i++) vol *= spatial[i];
  std::memset(out, 0, sizeof(float) * rb.size() * nPlanes * vol);
  float *oF = out;
  for (auto &r : rb) {
    Int nHot = (Int)(r.size() / 2);
    for (Int s = 0; s < nHot; s++) {
      const float *i = in + (size_t)r[2 * s] * nPlanes;
      float *o = oF + r[2 * s + 1];
      for (Int p = 0; p < nPlanes; p++) o[(size_t)p * vol] = i[p];
    }
    oF += (size_t)nPlanes * vol;
  }
}

// ---- point-at-a-time input (sparseconvnet/inputBatch.py over Metadata/Metadata.cpp:74-147,296-411)

// Metadata/Metadata.cpp:74-82
void orc_set_input_spatial_size(void *md, const int64_t *spatial) {
  Metadata &m = *(Metadata *)md;
  m.inputSpatialSize = mkkey(m.dim, spatial);
  m.grids[m.inputSpatialSize];
  m.nActive[m.inputSpatialSize];
}
// Metadata/Metadata.cpp:83-87
void orc_batch_add_sample(void *md) {
  Metadata &m = *(Metadata *)md;
  Grids &SGs = m.grids[m.inputSpatialSize];
  resize_grids(SGs, SGs.size() + 1, m.dim);
  m.currentSample = (Int)SGs.size() - 1;
}
// Metadata/Metadata.cpp:29-46: a new site takes the next row and the vector; a known site
// keeps its vector unless overwrite is set.
static void add_point(Metadata &m, Grid &mp, const Pt &p, const float *vec, int nPlanes, bool overwrite) {
  Int &nActive = m.nActive[m.inputSpatialSize];
  auto r = mp.insert(p, nActive);
  if (r.second) {
    nActive++;
    m.batchPlanes = nPlanes;
    m.batchFeatures.resize((size_t)nActive * nPlanes);
    std::memcpy(m.batchFeatures.data() + (size_t)(nActive - 1) * nPlanes, vec, sizeof(float) * nPlanes);
  } else if (overwrite) {
    std::memcpy(m.batchFeatures.data() + (size_t)*r.first * nPlanes, vec, sizeof(float) * nPlanes);
  }
}
// Metadata/Metadata.cpp:100-147: ncols == dim adds to the current sample, ncols == dim + 1
// reads the sample from the last column and grows the batch as needed.  Returns 0, or -1
// where the reference asserts (no current sample).
int orc_set_input_locations(void *md, const int64_t *locations, int n, int ncols, const float *vecs,
                            int nPlanes, int overwrite) {
  Metadata &m = *(Metadata *)md;
  Grids &SGs = m.grids[m.inputSpatialSize];
  if (ncols == m.dim && m.currentSample < 0) return -1;
  for (int i = 0; i < n; i++) {
    Pt p = Pt();
    for (int d = 0; d < m.dim; d++) p.x[d] = (Int)locations[(size_t)i * ncols + d];
    Int b = m.currentSample;
    if (ncols == m.dim + 1) {
      b = (Int)locations[(size_t)i * ncols + m.dim];
      if (b >= (Int)SGs.size()) resize_grids(SGs, b + 1, m.dim);
    }
    add_point(m, SGs[b], p, vecs + (size_t)i * nPlanes, nPlanes, overwrite != 0);
  }
  return 0;
}
// Metadata/Metadata.cpp:296-349: a new sample from a dense [size..., nPlanes] block placed at
// offset; a cell is active when some plane exceeds the threshold in magnitude and the cell
// lies inside the spatial size.  Cells are visited with the last dimension fastest
// (Metadata/RectangularRegions.h:84-91).
void orc_add_sample_from_tensor(void *md, const float *tensor, const int64_t *size, int nPlanes,
                                const int64_t *offset, float threshold) {
  Metadata &m = *(Metadata *)md;
  Grids &SGs = m.grids[m.inputSpatialSize];
  resize_grids(SGs, SGs.size() + 1, m.dim);
  Grid &sg = SGs.back();
  Int &nActive = m.nActive[m.inputSpatialSize];
  int64_t vol = 1;
  for (int d = 0; d < m.dim; d++) vol *= size[d];
  m.batchPlanes = nPlanes;
  Pt point = Pt();
  for (int d = 0; d < m.dim; d++) point.x[d] = (Int)offset[d];
  for (int64_t c = 0; c < vol; c++) {
    bool active = false;
    for (int i = 0; i < nPlanes; i++)
      if (std::fabs(tensor[i]) > threshold) {
        active = true;
        break;
      }
    for (int d = 0; d < m.dim; d++)
      if (point.x[d] < 0 || point.x[d] >= m.inputSpatialSize[d]) {
        active = false;
        break;
      }
    if (active) {
      *sg.insert(point, nActive).first = nActive;
      nActive++;
      m.batchFeatures.insert(m.batchFeatures.end(), tensor, tensor + nPlanes);
    }
    tensor += nPlanes;
    for (int d = m.dim - 1; d >= 0; d--) {
      point.x[d]++;
      if (point.x[d] < offset[d] + size[d]) break;
      point.x[d] = (Int)offset[d];
    }
  }
}
int orc_batch_planes(void *md) { return ((Metadata *)md)->batchPlanes; }
void orc_batch_features(void *md, float *out) {
  Metadata &m = *(Metadata *)md;
  if (!m.batchFeatures.empty()) std::memcpy(out, m.batchFeatures.data(), m.batchFeatures.size() * sizeof(float));
}
// Metadata/Metadata.cpp:351-411: every level's 3^d submanifold rulebook and the size-`size`
// stride-2 rulebook to the next level, until a level's extent no longer halves (size 2:
// even and >= 2; size 3: odd and >= 3).
void orc_generate_rulebooks(void *md, int size) {
  Metadata &m = *(Metadata *)md;
  int64_t inS[MAXD], outS[MAXD], s3[MAXD], sz[MAXD], str[MAXD];
  for (int d = 0; d < m.dim; d++) {
    inS[d] = m.inputSpatialSize[d];
    s3[d] = 3;
    sz[d] = size;
    str[d] = 2;
  }
  while (true) {
    getSubmanifoldRuleBook(m, inS, s3);
    for (int d = 0; d < m.dim; d++) {
      if (size == 2 ? (inS[d] < 2 || inS[d] % 2 != 0) : (inS[d] < 3 || inS[d] % 2 != 1)) return;
      outS[d] = size == 2 ? inS[d] / 2 : (inS[d] - 1) / 2;
    }
    getRuleBook(m, inS, outS, sz, str);
    for (int d = 0; d < m.dim; d++) inS[d] = outS[d];
  }
}

// ---- backward pass -------------------------------------------------------------------------

// The loop shared by CPU/Convolution.cpp:81-115 (strided), :152-185 (submanifold) and
// CPU/Deconvolution.cpp:43-77 (columns swapped).  d_in is zero-filled (:94-95), d_bias is the
// column sum of d_out when the input level has rows (:98-99); per offset with rules:
// d_w[k] = in_rows^T * d_out_rows (matmul_out, :109) and d_in_rows = d_out_rows * w[k]^T
// scatter-added (:110-111).  Offsets without rules leave d_w[k] as the caller made it; the
// Python side hands over zeros (submanifoldConvolution.py:101), and so does this function.
static void conv_backward_loop(const RuleBook &rules, int inCol, int outCol, const float *in, float *d_in,
                               Int nInRows, const float *d_out, Int nOutRows, const float *w, float *d_w,
                               float *d_bias, Int nIn, Int nOut, Int groups) {
  Int ip = nIn / groups, op = nOut / groups;
  std::memset(d_in, 0, sizeof(float) * (size_t)nInRows * nIn);
  std::memset(d_w, 0, sizeof(float) * rules.size() * (size_t)groups * ip * op);
  if (d_bias) {
    for (Int c = 0; c < nOut; c++) d_bias[c] = 0.f;
    if (nInRows)
      for (Int r = 0; r < nOutRows; r++)
        for (Int c = 0; c < nOut; c++) d_bias[c] += d_out[(size_t)r * nOut + c];
  }
  for (size_t k = 0; k < rules.size(); k++) {
    const auto &r = rules[k];
    Int nRules = (Int)(r.size() / 2);
    if (!nRules) continue;
    for (Int g = 0; g < groups; g++) {
      const float *wk = w + (((size_t)k * groups + g) * ip) * op;
      float *dwk = d_w + (((size_t)k * groups + g) * ip) * op;
      for (Int i = 0; i < nRules; i++) {
        const float *a = in + ((size_t)r[2 * i + inCol] * groups + g) * ip;
        const float *d = d_out + ((size_t)r[2 * i + outCol] * groups + g) * op;
        float *di = d_in + ((size_t)r[2 * i + inCol] * groups + g) * ip;
        for (Int c = 0; c < ip; c++) {
          float acc = 0.f;
          for (Int o = 0; o < op; o++) {
            dwk[(size_t)c * op + o] += a[c] * d[o];
            acc += d[o] * wk[(size_t)c * op + o];
          }
          di[c] += acc;
        }
      }
    }
  }
}
// CPU/Convolution.cpp:152-185
void orc_subm_conv_bwd(void *md, const int64_t *spatial, const int64_t *filter, const float *in, float *d_in,
                       const float *d_out, const float *w, float *d_w, float *d_bias, int nIn, int nOut,
                       int groups) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getSubmanifoldRuleBook(m, spatial, filter);
  Int n = m.nActive[mkkey(m.dim, spatial)];
  conv_backward_loop(rb, 0, 1, in, d_in, n, d_out, n, w, d_w, d_bias, nIn, nOut, groups);
}
// CPU/Convolution.cpp:81-115
void orc_conv_bwd(void *md, const int64_t *inSz, const int64_t *outSz, const int64_t *filter,
                  const int64_t *stride, const float *in, float *d_in, const float *d_out, const float *w,
                  float *d_w, float *d_bias, int nIn, int nOut, int groups) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getRuleBook(m, inSz, outSz, filter, stride);
  conv_backward_loop(rb, 0, 1, in, d_in, m.nActive[mkkey(m.dim, inSz)], d_out, m.nActive[mkkey(m.dim, outSz)], w,
                     d_w, d_bias, nIn, nOut, groups);
}
// CPU/Deconvolution.cpp:43-77: the rulebook of (outSz -> inSz); input rows are column 1.
void orc_deconv_bwd(void *md, const int64_t *inSz, const int64_t *outSz, const int64_t *filter,
                    const int64_t *stride, const float *in, float *d_in, const float *d_out, const float *w,
                    float *d_w, float *d_bias, int nIn, int nOut, int groups) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getRuleBook(m, outSz, inSz, filter, stride);
  conv_backward_loop(rb, 1, 0, in, d_in, m.nActive[mkkey(m.dim, inSz)], d_out, m.nActive[mkkey(m.dim, outSz)], w,
                     d_w, d_bias, nIn, nOut, groups);
}
// CPU/NetworkInNetwork.cpp:24-47: d_in = d_out * w^T; d_w = in^T * d_out; d_bias = column sums.
void orc_nin_bwd(const float *in, float *d_in, const float *d_out, const float *w, float *d_w, float *d_bias,
                 int nActive, int nIn, int nOut) {
  std::memset(d_in, 0, sizeof(float) * (size_t)nActive * nIn);
  std::memset(d_w, 0, sizeof(float) * (size_t)nIn * nOut);
  if (d_bias)
    for (int o = 0; o < nOut; o++) d_bias[o] = 0.f;
  for (int r = 0; r < nActive; r++) {
    const float *a = in + (size_t)r * nIn, *d = d_out + (size_t)r * nOut;
    for (int o = 0; o < nOut && d_bias; o++) d_bias[o] += d[o];
    for (int c = 0; c < nIn; c++) {
      float acc = 0.f;
      for (int o = 0; o < nOut; o++) {
        d_w[(size_t)c * nOut + o] += a[c] * d[o];
        acc += d[o] * w[(size_t)c * nOut + o];
      }
      d_in[(size_t)r * nIn + c] = acc;
    }
  }
}
// CPU/BatchNormalization.cpp:13-61 with train = true: batch statistics into saveMean /
// saveInvStd (sums of x and x*x in row order, :20-31), running statistics updated with
// `momentum` weighting the OLD value (:33-38, unbiased variance), then the affine map and the
// leaky ReLU as in eval mode.
void orc_bn_train(const float *in, float *out, int nActive, int nPlanes, int inStride, int outStride,
                  float *saveMean, float *saveInvStd, float *runningMean, float *runningVar,
                  const float *weight, const float *bias, float eps, float momentum, float leakiness) {
  std::memset(saveMean, 0, nPlanes * sizeof(float));
  std::memset(saveInvStd, 0, nPlanes * sizeof(float));
  for (int row = 0; row < nActive; row++)
    for (int p = 0; p < nPlanes; p++) {
      float v = in[(size_t)row * inStride + p];
      saveMean[p] += v;
      saveInvStd[p] += v * v;
    }
  for (int p = 0; p < nPlanes; p++) {
    saveMean[p] /= nActive;
    runningMean[p] = momentum * runningMean[p] + (1 - momentum) * saveMean[p];
    saveInvStd[p] -= saveMean[p] * saveMean[p] * nActive;
    runningVar[p] = momentum * runningVar[p] + (1 - momentum) * saveInvStd[p] / (nActive - 1);
    saveInvStd[p] = powf(saveInvStd[p] / nActive + eps, -0.5f);
  }
  for (int row = 0; row < nActive; row++)
    for (int p = 0; p < nPlanes; p++) {
      float wv = saveInvStd[p] * (weight ? weight[p] : 1.f);
      float bv = -saveMean[p] * wv + (bias ? bias[p] : 0.f);
      float v = in[(size_t)row * inStride + p] * wv + bv;
      out[(size_t)row * outStride + p] = v * ((v > 0) ? 1.f : leakiness);
    }
}
// CPU/BatchNormalization.cpp:63-107.  The reference scales d_out in place by the leaky slope
// (:79-81); here d_out is left alone and the scaled value is recomputed.
void orc_bn_bwd(const float *in, float *d_in, const float *out, const float *d_out, int nActive, int nPlanes,
                int inStride, int outStride, const float *saveMean, const float *saveInvStd,
                const float *weight, float *d_weight, float *d_bias, float leakiness) {
  std::vector<float> gradMean(nPlanes, 0.f), dotp(nPlanes, 0.f), k(nPlanes, 0.f);
  for (int row = 0; row < nActive; row++)
    for (int p = 0; p < nPlanes; p++) {
      float d = d_out[(size_t)row * outStride + p];
      d *= (out[(size_t)row * outStride + p] > 0) ? 1.f : leakiness;
      gradMean[p] += d;
      dotp[p] += (in[(size_t)row * inStride + p] - saveMean[p]) * d;
    }
  for (int p = 0; p < nPlanes; p++) {
    if (d_bias) d_bias[p] = gradMean[p];
    gradMean[p] /= nActive;
    k[p] = dotp[p] * saveInvStd[p] * saveInvStd[p] / nActive;
  }
  for (int row = 0; row < nActive; row++)
    for (int p = 0; p < nPlanes; p++) {
      float d = d_out[(size_t)row * outStride + p];
      d *= (out[(size_t)row * outStride + p] > 0) ? 1.f : leakiness;
      d_in[(size_t)row * inStride + p] = (d - gradMean[p] - (in[(size_t)row * inStride + p] - saveMean[p]) * k[p]) *
                                         saveInvStd[p] * (weight ? weight[p] : 1.f);
    }
  if (d_weight)
    for (int p = 0; p < nPlanes; p++) d_weight[p] = dotp[p] * saveInvStd[p];
}
// CPU/MaxPooling.cpp:21-35,61-87.  d_in is [rows(inSz), inStride], zero-filled.  As in the
// reference, the comparison reads the input planes WITHOUT the nFeaturesToDrop offset the
// forward pass applies (:77 against :55): with dropped features the gradient lands on the
// first nPlanes planes wherever they happen to equal the output.
void orc_maxpool_bwd(void *md, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                     const int64_t *stride, const float *in, float *d_in, int inStride, const float *out,
                     const float *d_out, int nPlanes, int nFeaturesToDrop) {
  (void)nFeaturesToDrop;
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getRuleBook(m, inSz, outSz, size, stride);
  std::memset(d_in, 0, sizeof(float) * (size_t)m.nActive[mkkey(m.dim, inSz)] * inStride);
  for (auto &r : rb)
    for (Int s = 0; s < (Int)(r.size() / 2); s++) {
      size_t i = (size_t)r[2 * s] * inStride, o = (size_t)r[2 * s + 1] * nPlanes;
      for (Int p = 0; p < nPlanes; p++)
        if (out[o + p] == in[i + p]) d_in[i + p] += d_out[o + p];
    }
}
// CPU/AveragePooling.cpp:21-35,62-86: d_in (zero-filled) [+ nFeaturesToDrop] += d_out / filterVolume.
void orc_avgpool_bwd(void *md, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                     const int64_t *stride, float *d_in, int inStride, const float *d_out, int nPlanes,
                     int nFeaturesToDrop) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getRuleBook(m, inSz, outSz, size, stride);
  std::memset(d_in, 0, sizeof(float) * (size_t)m.nActive[mkkey(m.dim, inSz)] * inStride);
  const Int filterVolume = (Int)rb.size();
  for (auto &r : rb)
    for (Int s = 0; s < (Int)(r.size() / 2); s++) {
      float *i = d_in + nFeaturesToDrop + (size_t)r[2 * s] * inStride;
      const float *o = d_out + (size_t)r[2 * s + 1] * nPlanes;
      for (Int p = 0; p < nPlanes; p++) i[p] += o[p] / filterVolume;
    }
}
// CPU/UnPooling.cpp:21-32,58-78: the rulebook of (outSz -> inSz); d_in lives on the coarse
// level inSz and is zero-filled by the caller (sparseconvnet/unPooling.py:49); here too.
void orc_unpool_bwd(void *md, const int64_t *inSz, const int64_t *outSz, const int64_t *size,
                    const int64_t *stride, float *d_in, int inStride, const float *d_out, int nPlanes,
                    int nFeaturesToDrop) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getRuleBook(m, outSz, inSz, size, stride);
  std::memset(d_in, 0, sizeof(float) * (size_t)m.nActive[mkkey(m.dim, inSz)] * inStride);
  for (auto &r : rb)
    for (Int s = 0; s < (Int)(r.size() / 2); s++) {
      float *i = d_in + nFeaturesToDrop + (size_t)r[2 * s + 1] * inStride;
      const float *o = d_out + (size_t)r[2 * s] * nPlanes;
      for (Int p = 0; p < nPlanes; p++) i[p] += o[p];
    }
}
// CPU/IOLayers.cpp:31-47 with the layer's own `average`: the gradient of every listed point.
static void input_backward_pass_avg(float *points, const float *rows, Int nRows, Int maxActive, int nPlanes,
                                    const Int *R, bool average) {
  for (Int row = 0; row < nRows; row++) {
    const Int *r = R + (size_t)row * (1 + maxActive);
    const float mult = (average && r[0] > 0) ? 1.f / r[0] : 1.f;
    const float *f = rows + (size_t)row * nPlanes;
    for (Int i = 1; i <= r[0]; ++i) {
      float *o = points + (size_t)r[i] * nPlanes;
      for (Int p = 0; p < nPlanes; p++) o[p] += mult * f[p];
    }
  }
}
// CPU/IOLayers.cpp:73-93.  d_in is [nInputRows, nPlanes].
void orc_input_bwd(void *md, float *d_in, const float *d_out, int nPlanes) {
  Metadata &m = *(Metadata *)md;
  auto &rules = m.inputLayerRuleBook;
  Int mode = rules[0][0], maxActive = rules[0][1], nRows = rules[0][3];
  if (mode == 0) {
    std::memcpy(d_in, d_out, sizeof(float) * (size_t)rules[0][2] * nPlanes);
    return;
  }
  std::memset(d_in, 0, sizeof(float) * (size_t)rules[0][2] * nPlanes);
  input_backward_pass_avg(d_in, d_out, nRows, maxActive, nPlanes, rules[1].data(), mode == 4);
}
// CPU/IOLayers.cpp:116-135: InputLayer_ForwardPass with average = false.  d_in is [nActive, nPlanes].
void orc_output_bwd(void *md, float *d_in, const float *d_out, int nPlanes) {
  Metadata &m = *(Metadata *)md;
  auto &rules = m.inputLayerRuleBook;
  Int mode = rules[0][0], maxActive = rules[0][1], nRows = rules[0][3];
  if (mode == 0) {
    std::memcpy(d_in, d_out, sizeof(float) * (size_t)rules[0][2] * nPlanes);
    return;
  }
  std::memset(d_in, 0, sizeof(float) * (size_t)nRows * nPlanes);
  input_forward_pass(d_out, d_in, nRows, maxActive, nPlanes, rules[1].data(), false);
}
// CPU/IOLayers.cpp:161-184.  d_in is [batchSize * length, nPlanes].
void orc_bl_input_bwd(void *md, float *d_in, const float *d_out, int nPlanes) {
  Metadata &m = *(Metadata *)md;
  auto &rules = m.blLayerRuleBook;
  Int mode = rules[0][0], maxActive = rules[0][1], nRows = rules[0][4];
  size_t nPoints = (size_t)rules[0][2] * rules[0][3];
  if (mode == 0) {
    std::memcpy(d_in, d_out, sizeof(float) * nPoints * nPlanes);
    return;
  }
  std::memset(d_in, 0, sizeof(float) * nPoints * nPlanes);
  input_backward_pass_avg(d_in, d_out, nRows, maxActive, nPlanes, rules[1].data(), mode == 4);
}
// CPU/IOLayers.cpp:207-229.  d_in is [nActive, nPlanes].
void orc_bl_output_bwd(void *md, float *d_in, const float *d_out, int nPlanes) {
  Metadata &m = *(Metadata *)md;
  auto &rules = m.blLayerRuleBook;
  Int mode = rules[0][0], maxActive = rules[0][1], nRows = rules[0][4];
  if (mode == 0) {
    std::memcpy(d_in, d_out, sizeof(float) * (size_t)nRows * nPlanes);
    return;
  }
  std::memset(d_in, 0, sizeof(float) * (size_t)nRows * nPlanes);
  input_forward_pass(d_out, d_in, nRows, maxActive, nPlanes, rules[1].data(), false);
}
// CPU/SparseToDense.cpp:21-33,66-90: d_in [nActive, nPlanes] = the dense gradient at every site.
void orc_s2d_bwd(void *md, const int64_t *spatial, float *d_in, const float *d_out, int nPlanes) {
  Metadata &m = *(Metadata *)md;
  RuleBook &rb = getSparseToDenseRuleBook(m, spatial);
  int64_t vol = 1;
  for (int i = 0; i < m.dim; i++) vol *= spatial[i];
  std::memset(d_in, 0, sizeof(float) * (size_t)m.nActive[mkkey(m.dim, spatial)] * nPlanes);
  const float *oF = d_out;
  for (auto &r : rb) {
    for (Int s = 0; s < (Int)(r.size() / 2); s++) {
      float *i = d_in + (size_t)r[2 * s] * nPlanes;
      const float *o = oF + r[2 * s + 1];
      for (Int p = 0; p < nPlanes; p++) i[p] = o[(size_t)p * vol];
    }
    oF += (size_t)nPlanes * vol;
  }
}

// Metadata/ActivePoolingRules.h:16-34 as its header comment describes it: rules[0] is a
// batchSize x (maxActive + 1) matrix, first column the number of active sites of the sample,
// then its rows (sg.ctr + value, in the grid's iteration order), zero padded.  (As written the
// reference pads with `while (rules.size() % (maxActive + 1) != 0)`, where rules.size() is the
// constant 2: that loop ends only when no sample has more than one site.  For such inputs this
// function and the reference agree; beyond, this is the matrix the comment specifies.)
static void active_pooling_rules(const Grids &SGs, std::vector<Int> &r, Int &maxActive) {
  maxActive = 0;
  for (auto &sg : SGs) maxActive = std::max(maxActive, (Int)sg.count);
  r.clear();
  for (auto &sg : SGs) {
    const size_t row0 = r.size();
    r.push_back((Int)sg.count);
    for (size_t b = 0; b < sg.used.size(); b++)
      if (sg.used[b]) r.push_back(sg.ctr + sg.vals[b]);
    r.resize(row0 + (size_t)maxActive + 1, 0);  // padding
  }
}
// CPU/ActivePooling.cpp:8-25,47-63: out [batchSize, nPlanes] = per sample the sum of its rows,
// times 1 / count with average.
// Returns 1 (the compiled reference's entry returns 0 where its rule builder would not return).
int orc_active_pooling(void *md, const int64_t *spatial, const float *in, float *out, int nPlanes, int average) {
  Metadata &m = *(Metadata *)md;
  const Grids &SGs = m.grids[mkkey(m.dim, spatial)];
  std::vector<Int> rules;
  Int maxActive = 0;
  active_pooling_rules(SGs, rules, maxActive);
  const Int batchSize = (Int)SGs.size();
  std::memset(out, 0, sizeof(float) * (size_t)batchSize * nPlanes);
  for (Int o = 0; o < batchSize; o++) {
    const Int *r = &rules[(size_t)o * (maxActive + 1)];
    Int nActive = *r++;
    const float mult = (average && nActive > 0) ? 1.0f / nActive : 1.0f;
    while (nActive-- > 0) {
      const float *inp = in + (size_t)(*r++) * nPlanes;
      for (int p = 0; p < nPlanes; p++) out[(size_t)o * nPlanes + p] += inp[p] * mult;
    }
  }
  return 1;
}
// CPU/ActivePooling.cpp:26-44,65-83: d_in [nActive, nPlanes]: every row receives its sample's
// gradient (times 1 / count with average).
int orc_active_pooling_bwd(void *md, const int64_t *spatial, float *d_in, const float *d_out, int nPlanes,
                           int average) {
  Metadata &m = *(Metadata *)md;
  const Grids &SGs = m.grids[mkkey(m.dim, spatial)];
  std::vector<Int> rules;
  Int maxActive = 0;
  active_pooling_rules(SGs, rules, maxActive);
  std::memset(d_in, 0, sizeof(float) * (size_t)m.nActive[mkkey(m.dim, spatial)] * nPlanes);
  for (Int o = 0; o < (Int)SGs.size(); o++) {
    const Int *r = &rules[(size_t)o * (maxActive + 1)];
    Int nActive = *r++;
    const float mult = (average && nActive > 0) ? 1.0f / nActive : 1.0f;
    while (nActive-- > 0) {
      float *inp = d_in + (size_t)(*r++) * nPlanes;
      for (int p = 0; p < nPlanes; p++) inp[p] = d_out[(size_t)o * nPlanes + p] * mult;
    }
  }
  return 1;
}

}  // extern "C"
