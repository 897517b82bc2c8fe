// Host-side state behind a scn_metadata handle: levels (one per spatial size), the input
// layer's rule lists and the cached neighbour tables.
#pragma once
#include <functional>
#include <map>
#include <memory>

#include "common.h"

namespace scn {

typedef std::vector<int64_t> SizeKey;

// One spatial size: which sites are active and where each row sits.
struct Level {
  Geom g{};
  int64_t n = 0;     // active sites
  int64_t npad = 0;  // n rounded up to 64: stride of the SoA arrays below
  int batch = 0;     // number of samples
  DevBuf<int> coords;                // [(dim+1)][npad]: coordinates, then sample index
  DevBuf<unsigned long long> keys;   // [n] site key of each row
  // Schedule: sched[t] = row, rows listed by ascending site key.  Kernels walk rows in
  // this order so that one workgroup's rows are neighbours in space whatever order the
  // caller's points came in.  Null when rows are already numbered by ascending key.
  DevBuf<int> sched;
  bool identity_sched = false;
  // Site lookup (common.h: BlockEntry), built on first use: block table, its mask (capacity
  // - 1, decided and kept on the device: gridp[0]) and the row of every distinct site in key
  // order.  `dups` marks levels whose keys may repeat (input-layer mode 0 with repeated
  // points: the last one wins, as with `mp[p] = i` in the reference); only those need `urow`,
  // elsewhere the u-th distinct site is schedule position u.
  DevBuf<BlockEntry> table;
  DevBuf<unsigned long long> gridp;
  DevBuf<int> urow;
  DevBuf<unsigned long long> skeys;  // [n + 1] site key of every schedule position (ascending); filled on first use
  bool skeys_ready = false;
  bool grid_built = false;
  bool dups = false;
  // Set when a strided rulebook makes the level: which construction of this spatial size it is
  // (a rulebook that still has to look its sites up checks that they are the ones it made).
  uint64_t gen = 0;
  // Active-site counts of the levels that successive filter 2 / stride 2 rulebooks make of this
  // one (size halved once, twice, ...), when somebody has computed them (metadata.hip:
  // halving_sizes): a strided build that finds its output size here needs no read-back.
  std::vector<int64_t> halvings;
  const int *urow_ptr() const { return dups ? urow.p : sched_ptr(); }
  const int *sched_ptr() const { return identity_sched ? nullptr : sched.p; }
};

// Neighbour table: nbr[k * npad + t] = row feeding filter tap k of the output row at
// position t, or -1; rowmap[t] = that output row.  Positions follow the level's schedule
// (ascending site key), then inside each of a few equal ranges of that order they are sorted
// by neighbour pattern (number of absent taps, then the bit mask of present taps), so that
// the positions a workgroup takes mostly need the same taps.  counts[k] = number of
// non-negative entries of tap k.
// Rule counts per tap of a rulebook.  They are tallied on the device while the rules are
// written and fetched only when somebody needs them on the host (multiply-add counts, list
// sizes of the export), so that building a rulebook needs no host round trip for them.  The
// two tables of a strided rulebook share one object; so do deferred multiply-add counts
// (Metadata::pending_macs), which is why it is held by shared_ptr.
struct Counts {
  int K = 0;
  int slots = 1;  // the device holds this many partial copies of the K counts, one after the other
  DevBuf<long long> dev;
  std::vector<int64_t> host;
  bool ready = false;  // host is valid
  int64_t total() const {
    int64_t s = 0;
    for (auto c : host) s += c;
    return s;
  }
};
void ensure_counts(Counts &c, hipStream_t s);  // fetches dev into host, summed over the copies (one stream synchronisation)

struct Table {
  int K = 0;
  int64_t n = 0, npad = 0;
  DevBuf<int> nbr;
  DevBuf<int> rowmap;
  DevBuf<unsigned> gmask;  // K <= 32 and pattern-sorted: bit k of gmask[i] = some position of granule i (16 positions) has tap k
  bool identity_rows = false;  // rowmap[t] == t: kernels skip the indirection
  // Tables with one rule per position (the fine side of a filter = stride = 2 rulebook): that rule
  // as (tap, row) of every position, in the table's order (few_tap[t] = 255: no rule); null elsewhere.
  DevBuf<unsigned char> few_tap;
  DevBuf<int> few_row;
  bool identity_few = false;  // the identity table: position t has the one rule (tap 0, row t); no arrays
  // The pattern sort ran over all positions at once (small levels): consecutive tiles descend in
  // cost from the first to the last, so kernels deal tiles to workgroups in turn instead of giving
  // each XCD a contiguous range.
  bool spread = false;
  const int *rowmap_ptr() const { return identity_rows ? nullptr : rowmap.p; }
  // Submanifold tables, decided on first use by a backward pass: does rule (k, i -> j) imply
  // rule (K-1-k, j -> i)?  (Odd filter sizes on a level without repeated points.)
  bool mirror_known = false, mirror = false;
  std::shared_ptr<Counts> cnt;  // never null once the table has been built
  const std::vector<int64_t> &counts(hipStream_t s) {
    ensure_counts(*cnt, s);
    return cnt->host;
  }
  int64_t total(hipStream_t s) {
    ensure_counts(*cnt, s);
    return cnt->total();
  }
};

struct StridedRules {
  Table by_out;  // indexed by rows of the coarse (output) level: value = fine row
  Table by_in;   // indexed by schedule positions of the fine level: value = coarse row
  // by_in is emitted with by_out but pattern-sorted only when somebody asks for it
  // (finish_by_in): transposed convolutions and unpooling come long after the level was built,
  // and the sort would sit on the path of the next level's construction.
  bool by_in_final = false;
  // Filter = stride = 2 over halving sizes: every fine position has at most one rule, kept as
  // (tap, coarse row) until finish_by_in writes the table in its sorted order (in_tap[t] < 0: no rule).
  bool by_in_compact = false;
  DevBuf<int> in_tap, in_row;
  // Rulebooks built by looking the fine sites up from the coarse ones (strided_rules: filters larger
  // than their stride): by_in does not exist until finish_by_in makes it the same way, from the
  // coarse level's site lookup; out_gen = Level::gen of the coarse level the rulebook made.
  bool by_in_lookup = false;
  uint64_t out_gen = 0;
  std::vector<int64_t> filter, stride;  // kept for that
  SizeKey in_size, out_size;
};

// A batch norm to fold to scale / shift arrays (device pointers); n_pad == 0: nothing to do.
struct CoefJob {
  const float *mean = nullptr, *var = nullptr, *gamma = nullptr, *beta = nullptr;
  float eps = 0.f;
  int n = 0, n_pad = 0;
  float *sc = nullptr, *sh = nullptr;
};
struct CoefJobs {
  CoefJob pre, post, post2;
};

// What a convolution derives from its parameters before it can run: the weights in MFMA operand
// order (one buffer per layout: the kernel taken depends on the level's size and on the bf16
// switch) and batch-norm statistics folded to scale / shift.  Normally derived on every call into
// the handle's scratch; a caller that knows its parameters unchanged between calls (inference)
// hands the convolution one of these objects to keep them in (scn_params_create).
struct FrozenParams {
  std::map<std::vector<int64_t>, DevBuf<float>> packed;
  DevBuf<float> pre, post, post2;   // scale | shift arrays, as conv_forward lays them out
  bool pre_done = false, post_done = false, post2_done = false;
  hipStream_t last = nullptr;  // the stream of the last convolution that used the set
  bool last_known = false;
  void clear() {
    packed.clear();
    pre.release();
    post.release();
    post2.release();
    pre_done = post_done = post2_done = false;
  }
};

struct InputRules {
  int mode = -1;      // 1: the first point of a site is listed, 2: the last, 3 / 4: all (sum / mean),
                      // 5: the first, unless later points of the site carry an overwrite flag: then the last of those
  int user_mode = -1; // the mode the caller gave (the batch-by-length layer numbers 1 and 2 the other way round)
  int max_active = 0;        // valid when max_known; read through input_max_active()
  bool max_known = true;     // false: the longest run is still in max_slots on the device (modes 3 and 4)
  DevBuf<int> max_slots;     // slotted maxima of the run lengths, written by the construction
  int64_t n_in = 0, n_out = 0;
  int64_t bl_batch = 0, bl_length = 0;  // batch-by-length input (BLInputLayer); 0: plain input layer
  DevBuf<int> row_of_input;  // [n_in]; -1: an empty position of a batch-by-length input
  DevBuf<int> sorted_idx;    // [n_in] input indices grouped by site, input order inside a group
  DevBuf<int> run_start;     // [n_out] first position of the row's group in sorted_idx
  DevBuf<int> run_len;       // [n_out]
  DevBuf<unsigned char> overwrite;  // [n_in], mode 5 only
};

// The one input point a site lists in modes 1, 2 and 5; [st, st + len) is the site's group in
// sorted_idx, in input order.
__device__ inline int listed_point(const int *sorted_idx, int st, int len, int mode, const unsigned char *overwrite) {
  if (mode == 2) return sorted_idx[st + len - 1];
  if (mode == 5)
    for (int q = len - 1; q > 0; q--) {
      const int i = sorted_idx[st + q];
      if (overwrite[i]) return i;
    }
  return sorted_idx[st];
}

// Where a construction reads the caller's coordinates: int64 as the caller holds them on the
// device, or the int16 / int32 values host_input.hip narrowed them to on their way from the host.
struct CoordSrc {
  const void *p;
  int width;  // bytes per value: 8, 4 or 2
};
__device__ inline int64_t coord_at(const CoordSrc &c, int64_t i) {
  if (c.width == 8) return static_cast<const int64_t *>(c.p)[i];
  if (c.width == 4) return static_cast<const int32_t *>(c.p)[i];
  return static_cast<const int16_t *>(c.p)[i];
}

// Pinned host blocks from a process-wide list (api.hip).
void *pinned_acquire(size_t bytes);
void pinned_release(void *p, size_t bytes);

struct Metadata {
  Metadata() = default;
  Metadata(const Metadata &) = delete;
  Metadata &operator=(const Metadata &) = delete;
  ~Metadata() {
    pinned_release(pinned, PINNED_WORDS * sizeof(int));
    if (staging) pinned_release(staging, staging_bytes);
  }
  // Coordinates that arrived in host memory: their narrowed copy on the device, and the pinned
  // block the copy was made from until the stream has been waited for (host_input.hip).
  DevBuf<unsigned char> hostcoords;
  void *staging = nullptr;
  size_t staging_bytes = 0;
  // Pinned host words that the constructions copy their sizes and flags into: a copy into
  // pageable memory would be staged and waited for by the runtime, one round trip per copy.
  static constexpr int PINNED_WORDS = 2048;
  int *pinned = nullptr;
  int dim = 0;
  std::map<SizeKey, Level> levels;
  InputRules input;
  SizeKey input_size;
  std::map<SizeKey, Table> subm;            // key: spatial || filter
  std::map<SizeKey, StridedRules> strided;  // key: in_size || filter || stride
  std::map<int64_t, Table> ident;           // key: rows; one tap, row t feeds row t (NetworkInNetwork)
  // scratch reused by the builders
  DevBuf<unsigned char> tmp;
  DevBuf<unsigned long long> k0, k1;
  DevBuf<int> v0, v1, f0, f1, s0, s1;
  DevBuf<float> wcols;  // column ranges of a wide layer's weights, one contiguous block per range (conv_forward)
  DevBuf<int> rowtab;  // site-major neighbour table on its way from the rule kernel to the pattern sort's permutation
  DevBuf<int> dflags;
  DevBuf<int> scan_tiles;  // exclusive_scan: the tiles' sums
  DevBuf<int> ob_words, ob_list, ob_part;  // strided rulebooks by lookup: counters, the coarse level's blocks, partial ranks
  uint64_t level_gen = 0;
  std::function<void()> before_pack;  // work the packing of the running convolution's weights needs first (the column-range path's copy), run at most once
  // while a column range of a wide layer runs: addresses in the scratch copy (from wkey_from) stand for
  // addresses from wkey_ptr in the caller's weights in a frozen set's keys
  int64_t wkey_ptr = 0, wkey_from = 0, wkey_c0 = 0, wkey_wc = 0;
  // a second output for the next convolution call (Epi::out2), with the batch norm it applies; serves one call
  float *next_out2 = nullptr;
  int64_t next_out2_stride = 0;
  const float *next_out2_bn[4] = {nullptr, nullptr, nullptr, nullptr};  // mean, var, gamma, beta
  float next_out2_eps = 0.f, next_out2_leak = 1.f;
  DevBuf<float> post2buf;
  int64_t next_out_stride = 0;  // floats between the output rows of the next convolution call (0: its plane count); serves one call
  DevBuf<unsigned long long> ticket;  // [0]: arrival ticket of grid_count (zero between launches), [1]: the count
  DevBuf<float> wpack;    // weights of the running convolution in MFMA operand order
  DevBuf<float> partial;  // partial tiles of a convolution whose taps are split over workgroups; partial sums of reductions
  DevBuf<float> wt;       // transposed weights of the input-gradient convolution of a backward pass
  DevBuf<int> queue;      // set counters of the resident-weights convolution kernel
  // The next convolution keeps its packed weights and folded batch norms here and takes what it
  // finds (scn_md_use_params; reset by every convolution call).
  FrozenParams *frozen = nullptr;
  bool queue_zeroed = false;  // `queue` has been cleared once (the kernel that uses it leaves it cleared)
  // Non-null while an allocation-free convolution runs: the three buffers above are then fixed
  // regions of a static device array (conv.hip) and nothing may be reserved.
  unsigned char *fixed_scratch = nullptr;
  // Multiply-add counts of forward calls that did not ask for theirs (macs == NULL): settled
  // ones summed, the others as (counts, multiply-adds per rule) until take_macs() fetches them.
  double macs_settled = 0;
  std::vector<std::pair<std::shared_ptr<Counts>, double>> pending_macs;
  int64_t cur_in_rows = 0;  // rows and start of the input matrix of the convolution being launched
  const float *cur_in_base = nullptr;
  CoefJobs jobs;          // coefficient arrays the next weight-packing launch has to fill
  CoefJob post_raw;       // the running convolution's batch norm behind it, for the kernel that folds it itself
  DevBuf<float> postbuf;  // scale / shift of a batch norm fused into the running convolution's stores
  DevBuf<float> prebuf;   // scale / shift of a batch norm fused into the running convolution
  DevBuf<float> bntmp;    // normalised input when a fused batch norm has no fused kernel
  // The row-owner and LDS-tiled convolution kernels (more than 32 output planes, or wide
  // inputs) round their operands to bf16 and run the bf16 MFMA with fp32 accumulation when the
  // input consists of whole 32-channel slabs; off unless the caller asks for it.
  bool bf16 = false;
  std::string last_kernel;  // what the last convolution call launched (scn_md_last_conv_kernel)
  // Ordering between the stream rulebooks are built on and the stream the caller's feature
  // passes run on (api.hip: BuildScope, consume).
  uint64_t builds = 0;              // bumped by every construction that enqueued work
  hipStream_t build_stream = nullptr;  // where the last construction ran (null: none yet)
  hipEvent_t ready[8] = {};         // ring of events recorded behind constructions
  int ready_next = 0;
  hipEvent_t last_ready = nullptr;  // what a feature pass has to wait for; null: nothing outstanding
  hipStream_t consumer = nullptr;   // the stream feature passes were last enqueued on ...
  bool consumer_known = false;
  bool consumer_waited = true;      // ... and whether it has been made to wait for last_ready
};

// Makes stream s wait for the feature passes enqueued so far on the caller's stream (before a
// construction overwrites or frees something they may still be reading).
void wait_for_consumers(Metadata &m, hipStream_t s);

SizeKey mk(int dim, const int64_t *a, const int64_t *b = nullptr, const int64_t *c = nullptr);
Geom make_geom(int dim, const int64_t *spatial);

// bl_length > 0: coords is [n / bl_length, bl_length, dim] (BLInputLayer), the sample is the
// first index and positions whose first coordinate is negative are empty.
// mode 5 (point-at-a-time input, Metadata/Metadata.cpp:29-46 as one pass): overwrite[i] != 0 marks
// points that replace what their site holds; NULL: none does.
void build_input_layer(Metadata &m, const int64_t *spatial, CoordSrc coords, int64_t n,
                       int ncols, int min_batch, int mode, hipStream_t s, int64_t bl_length = 0,
                       const unsigned char *overwrite = nullptr);
// host_input.hip
CoordSrc stage_host_coords(Metadata &m, const int64_t *host, int64_t values, hipStream_t s, bool allow16);
void release_staging(Metadata &m);
void generate_rulebooks(Metadata &m, int size, hipStream_t s);
void export_input_rules(Metadata &m, int *rows, hipStream_t s);
int input_max_active(Metadata &m);  // longest run of points on one site (modes 3 and 4), fetched from the device on first use
void spatial_locations(Metadata &m, const int64_t *spatial, int64_t *out, hipStream_t s);
Table &submanifold_rules(Metadata &m, const int64_t *spatial, const int64_t *filter, hipStream_t s);
StridedRules &strided_rules(Metadata &m, const int64_t *in_size, const int64_t *out_size,
                            const int64_t *filter, const int64_t *stride, hipStream_t s);
// The one-tap table over `rows` rows whose only rule list is the identity.
Table &identity_table(Metadata &m, int64_t rows, hipStream_t s);
void finish_by_in(Metadata &m, StridedRules &r, hipStream_t s);
// Pairs of tap k of a table: (value, row at position t), ordered by t.  Returns the count.
int64_t export_table_pairs(Metadata &m, Table &t, int k, bool swap, int *pairs, hipStream_t s);
std::vector<int64_t> s2d_sizes(Metadata &m, const int64_t *spatial, hipStream_t s);
int64_t export_s2d_pairs(Metadata &m, const int64_t *spatial, int sample, int *pairs,
                         hipStream_t s);

// What happens to an accumulated output value before it is stored: + bias, then optionally the
// eval batch norm + leaky ReLU of the layer that follows (folded to scale / shift per output
// channel), so that layer needs no pass of its own.
struct Epi {
  const float *bias = nullptr;               // [nOut] or null
  const float *sc = nullptr, *sh = nullptr;  // [nOut] each, or nulls
  float leak = 1.0f;
  int out_stride = 0;  // floats between output rows; 0: nOut
  // A second copy of the output before `sc` / `sh` are applied, with a batch norm of its own
  // (out2 == nullptr: none): out2[row * out2_stride + col] = act(value * sc2[col] + sh2[col]).
  float *out2 = nullptr;
  int out2_stride = 0;
  const float *sc2 = nullptr, *sh2 = nullptr;
  float leak2 = 1.0f;
};
// The second copy of one output value (raw: bias added, the convolution's own batch norm not yet).
__device__ inline void epi_second(const Epi &epi, int64_t row, int col, float raw);
__device__ inline float epi_act(float v, float sc, float sh, float leak) {
  const float y = v * sc + sh;
  return y > 0.f ? y : y * leak;
}
__device__ inline void epi_second(const Epi &epi, int64_t row, int col, float raw) {
  epi.out2[row * epi.out2_stride + col] = epi_act(raw, epi.sc2[col], epi.sh2[col], epi.leak2);
}
// Folding a batch norm to scale / shift (sc[c] = gamma / sqrt(var + eps), sh[c] = beta -
// mean * sc, zeros from n to n_pad) is a few hundred values: the weight-packing launch that
// precedes every MFMA convolution does it on the side (its first workgroup), so it costs no
// launch of its own.  CoefJobs lives in metadata.h.
__device__ inline void coef_job(const CoefJob &j) {
  for (int c = threadIdx.x; c < j.n_pad; c += blockDim.x) {
    float w = 0.f, b = 0.f;
    if (c < j.n) {
      w = (1.0f / sqrtf(j.var[c] + j.eps)) * (j.gamma ? j.gamma[c] : 1.0f);
      b = -j.mean[c] * w + (j.beta ? j.beta[c] : 0.0f);
    }
    j.sc[c] = w;
    j.sh[c] = b;
  }
}
__device__ inline void coef_jobs(const CoefJobs &jobs) {
  if (blockIdx.x != 0) return;
  if (jobs.pre.n_pad) coef_job(jobs.pre);
  if (jobs.post.n_pad) coef_job(jobs.post);
  if (jobs.post2.n_pad) coef_job(jobs.post2);
}
// conv_first.hip: the convolution kernel for nIn <= 4, nOut <= 32 and up to 32 taps; it reads the
// weights as the caller holds them and folds the batch norm behind the convolution itself
// (bn.n == 0: none), so it needs no scratch.  in_rows: rows of the input matrix that starts at `in`.
bool conv_first_serves(const Table &t, int64_t in_rows, int n_in, int n_out);
void conv_first_forward(const Table &t, const float *in, int64_t in_rows, float *out, const float *w, const float *bias,
                        CoefJob bn, float leak, int n_in, int n_out, hipStream_t s);

// sort.hip: stable radix sort of (key, value) pairs by the low end_bit bits of the key; the input
// arrays are left as they are, scratch comes from m.tmp.
void radix_sort_pairs(Metadata &m, const unsigned long long *kin, unsigned long long *kout, const int *vin, int *vout,
                      int64_t n, int end_bit, hipStream_t s, const int *n_dev = nullptr);

// ops.hip / conv.hip
unsigned char *noalloc_scratch();  // the static scratch array's address on the current device
void fill32(void *p, uint32_t v, int64_t n, hipStream_t s);
struct BnArgs {  // eval batch norm + leaky ReLU in front of a convolution (device pointers)
  const float *mean, *var, *gamma, *beta;
  float eps, leak;
};
void note_macs(Metadata &m, Table &t, double per_rule, double *macs, hipStream_t s);
double take_macs(Metadata &m, hipStream_t s);
void conv_forward(Metadata &m, const Table &t, const float *in, int64_t n_in_rows, float *out, const float *w,
                  const float *bias, int n_in, int n_out, int groups, const BnArgs *bn, const BnArgs *post,
                  hipStream_t s);
void maxpool_forward(const Table &t, const float *in, int in_stride, float *out, int planes,
                     int drop, hipStream_t s);
void avgpool_forward(const Table &t, const float *in, int in_stride, float *out, int planes,
                     int drop, hipStream_t s);
void unpool_forward(const Table &t, const float *in, int in_stride, float *out, int planes,
                    int drop, hipStream_t s);
void bn_eval_forward(const float *in, float *out, int64_t rows, int planes, int64_t in_stride,
                     int64_t out_stride, const float *mean, const float *var, const float *gamma,
                     const float *beta, float eps, float leak, hipStream_t s);
void input_forward(const InputRules &r, const float *in, float *out, int planes, hipStream_t s);
void output_forward(const InputRules &r, const float *in, float *out, int planes, hipStream_t s);
void s2d_forward(const Level &l, const float *in, float *out, int planes, hipStream_t s);
void active_pool_forward(Metadata &m, const Level &l, const float *in, float *out, int planes, int average, hipStream_t s);
void active_pool_backward(Metadata &m, const Level &l, float *d_in, const float *d_out, int planes, int average,
                          hipStream_t s);

// backward.hip
void subm_conv_backward(Metadata &m, Table &t, const int64_t *filter, const float *in, float *d_in,
                        const float *d_out, const float *w, float *d_w, float *d_bias, int n_in, int n_out,
                        int groups, hipStream_t s);
void strided_conv_backward(Metadata &m, const Table &fwd, const Table &other, int64_t in_rows, int64_t out_rows,
                           const float *in, float *d_in, const float *d_out, const float *w, float *d_w, float *d_bias,
                           int n_in, int n_out, int groups, hipStream_t s);
void nin_backward(Metadata &m, const Table &t, const float *in, float *d_in, const float *d_out, const float *w,
                  float *d_w, float *d_bias, int n_in, int n_out, hipStream_t s);
void bn_train_forward(Metadata *scratch, const float *in, float *out, int64_t rows, int planes, int64_t in_stride,
                      int64_t out_stride, float *save_mean, float *save_invstd, float *running_mean,
                      float *running_var, const float *gamma, const float *beta, float eps, float momentum,
                      float leak, hipStream_t s);
void bn_backward(Metadata *scratch, const float *in, float *d_in, const float *out, const float *d_out, int64_t rows,
                 int planes, int64_t in_stride, int64_t out_stride, const float *save_mean, const float *save_invstd,
                 const float *gamma, float *d_gamma, float *d_beta, float leak, hipStream_t s);
// mode 0: max pooling (table read from the fine side), 1: average pooling (fine side), 2: unpooling (coarse side)
void pool_backward(int mode, const Table &t, const float *in, float *d_in, int in_stride, const float *out,
                   const float *d_out, int planes, int drop, hipStream_t s);
void s2d_backward(const Level &l, float *d_in, const float *d_out, int planes, hipStream_t s);
void input_backward(const InputRules &r, float *d_in, const float *d_out, int planes, hipStream_t s);
void output_backward(const InputRules &r, float *d_in, const float *d_out, int planes, hipStream_t s);

}  // namespace scn
