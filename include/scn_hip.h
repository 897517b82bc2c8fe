/* C ABI of libscn_hip.so: the MI355X (gfx950) path of submanifold sparse
 * convolutional networks (forward pass, and the backward pass of the same ops).
 *
 * The library replaces what the reference binds through its pybind11 module
 * `sparseconvnet.SCN` for the forward pass (reference paths are relative to
 * sparseconvnet/SCN/): the `Metadata_<D>` class (pybind.cpp:11-33,
 * Metadata/Metadata.h:44-167) and the `*_updateOutput` functions declared in
 * sparseconvnet.h:22-246.  Signatures carry plain pointers and sizes only.
 *
 * Conventions
 *  - every function returns 0 on success, non-zero on failure; the message is
 *    read with scn_last_error() (thread-local).  The reference has no error
 *    codes: its shape checks are Python asserts and C++ asserts.
 *  - `spatial`, `filter`, `stride` arguments are HOST arrays of `dim` int64
 *    (the reference passes 1-D CPU LongTensors, Metadata/32bits.h:17-24).
 *  - feature / weight / coordinate pointers are DEVICE pointers; features are
 *    fp32 row-major [rows, planes]; weights [K, groups, nIn/groups,
 *    nOut/groups] as in sparseconvnet/submanifoldConvolution.py:24-26.
 *  - outputs are allocated by the caller (the reference resizes the tensor it
 *    is handed, CPU/Convolution.cpp:127): ask scn_md_nactive() for the row count
 *    after the rulebook call that creates the level.
 *  - `stream` is a hipStream_t (as void*); work is enqueued on it.  Calls that
 *    return a host value (row counts, rule counts) synchronise that stream.
 *  - a metadata handle is not thread-safe (neither is the reference's lazily
 *    caching Metadata, Metadata/Metadata.cpp:442-449).
 */
#ifndef SCN_HIP_H
#define SCN_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct scn_metadata scn_metadata;

/* Message of the last failure on the calling thread ("" if none). */
const char *scn_last_error(void);
/* 32: rule indices are int32, as the reference's n_rulebook_bits (pybind.cpp:235). */
int scn_rulebook_bits(void);

/* ---- Metadata (pybind.cpp:11-33; Metadata/Metadata.h:44-167) ------------ */

/* Metadata_<dim>() constructor, dim in 1..6 (pybind.cpp:204-209). NULL on failure. */
scn_metadata *scn_md_create(int dim);
void scn_md_destroy(scn_metadata *md);
/* Metadata::clear (Metadata/Metadata.cpp:52-66). */
int scn_md_clear(scn_metadata *md);

/* Rulebooks depend on coordinates only.  By default the library builds them on a stream of its
 * own (one per device, default priority) and orders that stream against the stream argument of
 * each call with events, so that the construction of the next level's rulebook runs beside the
 * convolutions already enqueued: a new scene's forward pass then costs little more than its
 * convolutions.  Results are the same either way.  enable = 0 builds on the caller's stream
 * (also: SCN_BUILD_STREAM=0 in the environment); returns the previous setting.  Process-wide;
 * affects constructions started afterwards.  No counterpart in the reference, whose rulebooks
 * are built on the host. */
int scn_set_build_stream(int enable);
/* Optional reduced-precision path (no counterpart in the reference, which computes in fp32
 * throughout): with enable != 0 the convolutions of this handle whose input rows consist of
 * whole 32-channel slabs and that run in the two wide kernel families (more than 32 output
 * planes, or 128 and more input planes) round input rows and weights to bf16 (nearest even)
 * and use the bf16 MFMA with fp32 accumulation; outputs, batch norms and everything else stay
 * fp32.  Results then agree with the fp32 path to about 1e-2 relative to the output scale.
 * Off by default. */
int scn_md_set_bf16(scn_metadata *md, int enable);
/* No counterpart in the reference: the kernel the handle's last convolution call ran, as text
 * (family and tile shape, e.g. "rows ncb=6 rg=1 ss=2 nw=4 split=1"), for benchmark tables and
 * profiles.  The pointer stays valid until the handle's next convolution call. */
const char *scn_md_last_conv_kernel(scn_metadata *md);
/* No counterpart in the reference (its JoinTable copies, sparseconvnet/tables.py:35-48): the next
 * convolution call on this handle (scn_subm_conv_fwd, scn_conv_fwd, scn_deconv_fwd, scn_conv_bn_fwd,
 * scn_nin_fwd) writes its output rows `stride` floats apart instead of nOut, so that a caller can
 * have it fill a range of columns of a wider matrix (the part of a concatenation that the
 * convolution produces).  stride >= nOut, nOut <= 256; it serves one call and 0 switches it off. */
int scn_md_next_output_stride(scn_metadata *md, int64_t stride);
/* Metadata::inputLayer (Metadata/Metadata.cpp:413-425, Metadata/IOLayersRules.h:18-121).
 * coords: device int64 [n, ncols], ncols = dim (one sample) or dim+1 (last column = sample
 * index).  mode 0: rows = input order, no merging; 1: first, 2: last, 3: sum, 4: mean of the
 * points that share a site; rows are numbered by first occurrence in input order.
 * min_batch is the reference's batchSize argument (a lower bound on the number of samples).
 * Coordinates outside [0, spatial) are an error (the reference leaves them undefined).
 * Writes the number of active sites to *n_active. */
int scn_md_input_layer(scn_metadata *md, const int64_t *spatial, const int64_t *coords,
                       int64_t n, int ncols, int min_batch, int mode, void *stream,
                       int64_t *n_active);
/* The same with the coordinates in host memory, as the reference's InputLayer receives them (a CPU
 * LongTensor, sparseconvnet/ioLayers.py:51-65; Metadata/Metadata.cpp:413-425 reads it on the host).
 * coords: host int64 [n, ncols], pageable or pinned; it has been read completely when the call
 * returns.  A few host threads narrow the values to int16 (grids of up to 32767 cells per
 * dimension; int32 otherwise or when a value does not fit) into pinned memory and the pieces are
 * copied while the next ones are narrowed: a quarter of the bytes of an int64 copy cross PCIe. */
int scn_md_input_layer_host(scn_metadata *md, const int64_t *spatial, const int64_t *host_coords,
                            int64_t n, int ncols, int min_batch, int mode, void *stream,
                            int64_t *n_active);
/* The point-at-a-time input of sparseconvnet/inputBatch.py, as one pass over everything the
 * caller collected: Metadata::setInputSpatialSize / batchAddSample / setInputSpatialLocation(s)
 * (Metadata/Metadata.cpp:74-147) with addPointToSparseGridMapAndFeatures (:29-46).  coords as
 * for scn_md_input_layer, in the order the points were set; a site's row is the rank of its
 * first point, and the site lists that point unless later points of the site have
 * overwrite[i] != 0: then it lists the last of those (overwrite: device bytes [n], or NULL for
 * "no point overwrites"; copied, so the caller may free it).  min_batch is the number of
 * samples added so far (samples without points count).  scn_input_layer_fwd then gathers the
 * listed points' vectors into the [n_active, planes] feature matrix the reference grows row by
 * row.  scn_md_input_rules_header reports mode 5 (1 without flags), maxActive 1. */
int scn_md_input_batch(scn_metadata *md, const int64_t *spatial, const int64_t *coords,
                       const unsigned char *overwrite, int64_t n, int ncols, int min_batch,
                       void *stream, int64_t *n_active);
/* Metadata::generateRuleBooks2s2 / generateRuleBooks3s2 (Metadata/Metadata.cpp:351-411;
 * InputBatch.precompute_metadata, sparseconvnet/inputBatch.py:72-82): starting at the input
 * level, every level's 3^d submanifold rulebook and the size-`size` (2 or 3), stride-2 rulebook
 * to the next level, until an extent no longer halves (size 2: even and >= 2; size 3: odd and
 * >= 3).  Everything is enqueued on the library's build stream (see scn_set_build_stream); later
 * calls that use one of the rulebooks wait for it there. */
int scn_md_generate_rulebooks(scn_metadata *md, int size, void *stream);
/* Rule header [mode, maxActive, nInputRows, nOutputRows] (Metadata/IOLayersRules.h:10-15). */
int scn_md_input_rules_header(scn_metadata *md, int32_t hdr[4]);
/* Rule rows, device int32 [nOutputRows, 1+maxActive] = [count, input indices.., 0 pad]. */
int scn_md_input_rules(scn_metadata *md, int32_t *rows, void *stream);
/* Metadata::blLayer (Metadata/Metadata.cpp:426-436, Metadata/IOLayersRules.h:132-286), the rule
 * half of BLInputLayer_updateOutput (pybind.cpp:168-173 region, CPU/IOLayers.cpp:117-139).
 * coords: device int64 [batch, length, dim]; a position whose first coordinate is negative is
 * empty.  Sample b holds positions b*length .. (b+1)*length-1; rows are numbered by first
 * occurrence, sample after sample.  mode 0: every position is a row of its own (none may be
 * empty); 1: the last point of a site, 2: the first (the opposite of scn_md_input_layer, as
 * in the reference); 3: sum; 4: mean.  The feature passes are scn_input_layer_fwd
 * (in [batch*length, planes]) and scn_output_layer_fwd (out [batch*length, planes], zeros at
 * empty positions: BLOutputLayer_updateOutput, CPU/IOLayers.cpp:186-206); the rule rows come
 * from scn_md_input_rules. */
int scn_md_bl_input_layer(scn_metadata *md, const int64_t *spatial, const int64_t *coords,
                          int64_t batch, int64_t length, int mode, void *stream,
                          int64_t *n_active);
/* Rule header [mode, maxActive, batchSize, length, nOutputRows] (Metadata/IOLayersRules.h:122-128). */
int scn_md_bl_rules_header(scn_metadata *md, int32_t hdr[5]);

/* Metadata::getNActive (Metadata/Metadata.cpp:67-70); 0 for an unknown level. */
int scn_md_nactive(scn_metadata *md, const int64_t *spatial, int64_t *n_active);
/* Metadata::getBatchSize (Metadata/Metadata.cpp:171-176). */
int scn_md_batch_size(scn_metadata *md, const int64_t *spatial, int *batch);
/* Metadata::getSpatialLocations (Metadata/Metadata.cpp:149-170): device int64
 * [nActive, dim+1], coordinates then sample index. */
int scn_md_spatial_locations(scn_metadata *md, const int64_t *spatial, int64_t *out,
                             void *stream);

/* Metadata::getSubmanifoldRuleBook (Metadata/Metadata.cpp:437-451,
 * Metadata/SubmanifoldConvolutionRules.h:11-87): builds and caches the rulebook of
 * (spatial, filter).  Idempotent. */
int scn_md_submanifold_rules(scn_metadata *md, const int64_t *spatial, const int64_t *filter,
                             void *stream);
/* Metadata::getRuleBook (Metadata/Metadata.cpp:492-518, Metadata/ConvolutionRules.h:11-105):
 * builds and caches the rulebook of (in_size, filter, stride) and, as the reference does,
 * REPLACES the level out_size with the sites the rules reach.  Rows of that level are
 * numbered by sample, then along a space-filling curve (the reference's order is its hash
 * map's bucket order; both are arbitrary, compare through scn_md_spatial_locations). */
int scn_md_strided_rules(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                         const int64_t *filter, const int64_t *stride, void *stream);

/* Rule export, for inspection and parity tests (the reference binds no rulebook getter;
 * its lists are the RuleBook vectors of Metadata/Metadata.h:35).
 * kind 0: submanifold (a=spatial, b=filter); kind 1: strided (a=in_size, b=out_size,
 * c=filter, d=stride); kind 2: sparse-to-dense (a=spatial; one list per sample of
 * (row, dense offset), Metadata/ConvolutionRules.h:130-151).  Builds the rulebook if needed.
 * scn_rules_count: number of lists.  scn_rules_sizes: host int64[count] pairs per list.
 * scn_rules_export: device int32 [sizes[k], 2] (first, second) pairs of list k. */
int scn_rules_count(scn_metadata *md, int kind, const int64_t *a, const int64_t *b,
                    const int64_t *c, const int64_t *d, void *stream, int *count);
int scn_rules_sizes(scn_metadata *md, int kind, const int64_t *a, const int64_t *b,
                    const int64_t *c, const int64_t *d, void *stream, int64_t *sizes);
int scn_rules_export(scn_metadata *md, int kind, const int64_t *a, const int64_t *b,
                     const int64_t *c, const int64_t *d, int k, int32_t *pairs, void *stream);
/* ---- forward ops (sparseconvnet.h:22-246) -------------------------------- */

/* The convolution calls below return the multiply-add count the reference returns
 * (CPU/Convolution.cpp:141) through `macs`; the first time a rulebook is used that costs a
 * stream synchronisation (the rule counts are tallied on the device).  A caller that passes
 * macs = NULL has the count added to a per-metadata total instead, which this call returns
 * and resets (one synchronisation for everything that is still outstanding): asked once,
 * after a network has been enqueued, it keeps the GPU busy in between.  The reference has no
 * counterpart; its Python layer sums the per-call values (sparseconvnet/__init__.py:7). */
int scn_md_take_macs(scn_metadata *md, void *stream, double *macs);
/* A handle that is destroyed or cleared while it still owes such a total does not wait for the
 * GPU: its rule counts are copied to pinned memory behind the work already enqueued.  This call
 * waits for those copies and returns (and resets) the multiply-adds of all handles that are
 * gone.  No counterpart in the reference. */
int scn_take_released_macs(double *macs);

/* The library's own device buffers (rulebooks, levels, scratch) come from a process-wide cache
 * of blocks that outlive the handle that used them, so that a stream of scenes does no
 * hipMalloc / hipFree.  scn_release_cache waits for the device and gives every idle block back
 * to the driver (call it when another allocator in the process runs out of memory);
 * scn_cache_stats reports bytes in use by live handles, idle bytes held, the high-water mark of
 * their sum and the number of hipMalloc calls made so far (any pointer may be NULL).  No
 * counterpart in the reference, whose rulebooks live in host memory. */
int scn_release_cache(void);
int scn_cache_stats(int64_t *live_bytes, int64_t *idle_bytes, int64_t *peak_bytes,
                    int64_t *device_allocations);

/* The sort the rulebook builders use, by itself (for tests and measurement): a stable sort of
 * n (64-bit key, 32-bit value) pairs, device arrays, by the low end_bit bits of the key; the
 * input arrays are not written, scratch comes from the handle.  The reference keeps its sites
 * in hash maps and has no such step (Metadata/Metadata.h:22-33). */
int scn_sort_pairs(scn_metadata *md, const unsigned long long *keys_in, unsigned long long *keys_out,
                   const int *values_in, int *values_out, int64_t n, int end_bit, void *stream);

/* InputLayer_updateOutput after the rules exist (pybind.cpp:155-159, CPU/IOLayers.cpp:49-72):
 * in [nInputRows, planes] -> out [nActive, planes]. */
int scn_input_layer_fwd(scn_metadata *md, const float *in, float *out, int planes, void *stream);
/* OutputLayer_updateOutput (pybind.cpp:164-167, CPU/IOLayers.cpp:95-115):
 * in [nActive, planes] -> out [nInputRows, planes]. */
int scn_output_layer_fwd(scn_metadata *md, const float *in, float *out, int planes,
                         void *stream);

/* SubmanifoldConvolution_updateOutput (pybind.cpp:135-139, CPU/Convolution.cpp:117-150).
 * in [nActive, nIn] -> out [nActive, nOut]; bias may be NULL; *macs receives the
 * multiply-add count the reference returns (CPU/Convolution.cpp:141); macs may be NULL. */
int scn_subm_conv_fwd(scn_metadata *md, const int64_t *spatial, const int64_t *filter,
                      const float *in, float *out, const float *weight, const float *bias,
                      int n_in, int n_out, int groups, void *stream, double *macs);
/* scn_subm_conv_fwd for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and result as scn_subm_conv_fwd with groups = 1 (the result may
 * differ in the order of fp32 additions: small levels split their taps over fewer workgroups
 * when the partial sums would not fit), but the call performs no hipMalloc / hipFree: the
 * kernels' scratch (weights in MFMA operand order, work counters, partial tiles) lives in a
 * static 16 MiB device array that every GPU the library runs on holds until the process ends.
 * Limits: the rulebook of (spatial, filter) must exist already (scn_md_submanifold_rules, or an
 * earlier convolution); the packed weights, filter volume x ceil(n_in/16)*16 x ceil(n_out/16)*16
 * x 4 bytes, must fit in 8 MiB (27 taps of 256 x 256 do), and n_out may be at most 256 (wider
 * layers would need an allocated copy of their weights), else the call fails with a message.
 * All such calls on one GPU share the array: calls that overlap on one GPU (two streams, two
 * threads) race; calls on one stream are ordered.  The multiply-add count is added to the
 * handle's running total (scn_md_take_macs). */
int scn_subm_conv_fwd_noalloc(scn_metadata *md, const int64_t *spatial, const int64_t *filter,
                              const float *in, float *out, const float *weight, const float *bias,
                              int n_in, int n_out, void *stream);
/* Convolution_updateOutput (pybind.cpp:55-60, CPU/Convolution.cpp:45-79).
 * in [nActive(in_size), nIn] -> out [nActive(out_size), nOut]. */
int scn_conv_fwd(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                 const int64_t *filter, const int64_t *stride, const float *in, float *out,
                 const float *weight, const float *bias, int n_in, int n_out, int groups,
                 void *stream, double *macs);
/* Deconvolution_updateOutput (pybind.cpp:79-84, CPU/Deconvolution.cpp:7-41): uses the
 * rulebook of (out_size -> in_size) with its columns swapped.
 * in [nActive(in_size), nIn] -> out [nActive(out_size), nOut]. */
int scn_deconv_fwd(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                   const int64_t *filter, const int64_t *stride, const float *in, float *out,
                   const float *weight, const float *bias, int n_in, int n_out, int groups,
                   void *stream, double *macs);
/* A convolution with the eval-mode batch norms + leaky ReLUs next to it folded in:
 * BatchNormalization_updateOutput(train=false) (pybind.cpp:220, CPU/BatchNormalization.cpp:41-61)
 * of the layer in front (`pre`, over the n_in input planes, applied while the input rows are
 * gathered) and / or of the layer behind (`post`, over the n_out output planes, applied as the
 * output rows are stored), so that neither layer reads and writes the feature matrix itself.
 * Every block of the reference's U-Net is such a pair (networkArchitectures.py:232-234).
 * kind 0: SubmanifoldConvolution (a = spatial, b = filter, c = d = NULL); 1: Convolution,
 * 2: Deconvolution (a = in_size, b = out_size, c = filter, d = stride); the other arguments
 * are those of the plain calls.  pre / post may be NULL.  Results equal the separate calls up
 * to fp32 rounding. */
typedef struct scn_bn_params {
  const float *running_mean, *running_var; /* device, [planes] */
  const float *gamma, *beta;               /* device, [planes], or NULL */
  float eps, leakiness;
} scn_bn_params;
/* No counterpart in the reference: the next convolution call on this handle also writes a second
 * copy of its output, taken before the batch norm behind the convolution (if any) is applied and
 * normalised with `bn` instead: out2[row * stride + col] = leaky(bn(value)).  For a producer whose
 * plain output feeds one consumer and whose normalised output is one part of a concatenation
 * (the skip connection of a U-Net level, sparseconvnet/networkArchitectures.py:240-253): the
 * part lands in its columns of the joined matrix without a pass of its own.  groups = 1,
 * nOut <= 256, stride >= nOut; serves one call; out2 = NULL switches it off. */
int scn_md_next_second_output(scn_metadata *md, float *out2, int64_t stride, const scn_bn_params *bn);
int scn_conv_bn_fwd(scn_metadata *md, int kind, const int64_t *a, const int64_t *b,
                    const int64_t *c, const int64_t *d, const float *in, float *out,
                    const float *weight, const float *bias, int n_in, int n_out, int groups,
                    const scn_bn_params *pre, const scn_bn_params *post, void *stream,
                    double *macs);
/* NetworkInNetwork_updateOutput (pybind.cpp:225, sparseconvnet.h:51-54, CPU/NetworkInNetwork.cpp:7-23):
 * out [rows, n_out] = bias + in [rows, n_in] * weight [n_in, n_out]; a convolution with one
 * tap.  The reference call takes no metadata; here the handle of the tensor's metadata owns
 * the scratch the kernels use (packed weights, the one-tap table for this row count), which
 * the caller has at hand (SparseConvNetTensor.metadata).  macs as for the convolutions
 * (rows * n_in * n_out). */
int scn_nin_fwd(scn_metadata *md, const float *in, float *out, const float *weight,
                const float *bias, int64_t rows, int n_in, int n_out, void *stream,
                double *macs);
/* MaxPooling_updateOutput (pybind.cpp:103-107, CPU/MaxPooling.cpp:37-60).
 * in [nActive(in_size), in_stride] -> out [nActive(out_size), planes] where
 * planes = in_stride - n_features_to_drop; the result is max(0, inputs of the window). */
int scn_maxpool_fwd(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                    const int64_t *size, const int64_t *stride, const float *in, int in_stride,
                    float *out, int planes, int n_features_to_drop, void *stream);
/* AveragePooling_updateOutput (pybind.cpp:44-48, sparseconvnet.h:74-78,
 * CPU/AveragePooling.cpp:38-61): as scn_maxpool_fwd, the result is the sum of the window's
 * active inputs divided by the filter volume (absent sites count as zeros). */
int scn_avgpool_fwd(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                    const int64_t *size, const int64_t *stride, const float *in, int in_stride,
                    float *out, int planes, int n_features_to_drop, void *stream);
/* UnPooling_updateOutput (pybind.cpp:189-193, sparseconvnet.h:230-234, CPU/UnPooling.cpp:34-57):
 * in [nActive(in_size), in_stride] on the coarse level -> out [nActive(out_size), planes] on
 * the finer level out_size, which must exist already (as for scn_deconv_fwd): every fine site
 * receives the sum of the coarse rows whose windows hold it. */
int scn_unpool_fwd(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                   const int64_t *size, const int64_t *stride, const float *in, int in_stride,
                   float *out, int planes, int n_features_to_drop, void *stream);
/* BatchNormalization_updateOutput with train=false (pybind.cpp:220,
 * CPU/BatchNormalization.cpp:41-61,109-130): out = leaky(x*w + b), w = gamma/sqrt(var+eps),
 * b = beta - mean*w.  gamma/beta may be NULL.  Row strides in elements. */
int scn_bn_eval_fwd(const float *in, float *out, int64_t rows, int planes, int64_t in_stride,
                    int64_t out_stride, const float *running_mean, const float *running_var,
                    const float *gamma, const float *beta, float eps, float leakiness,
                    void *stream);
/* SparseToDense_updateOutput (pybind.cpp:125-129, CPU/SparseToDense.cpp:35-64):
 * in [nActive, planes] -> out [batch, planes, spatial...], zero-filled first. */
int scn_s2d_fwd(scn_metadata *md, const int64_t *spatial, const float *in, float *out,
                int planes, void *stream);

/* Parameters that do not change between calls (inference).  A convolution call derives two things
 * from its parameters before it can run: the weights in the operand order of the matrix
 * instructions, and each fused batch norm folded to scale / shift; by default on every call.  A
 * scn_params object keeps them: scn_md_use_params(md, p) makes the NEXT convolution call on md
 * (scn_subm_conv_fwd, scn_conv_fwd, scn_deconv_fwd, scn_conv_bn_fwd, scn_nin_fwd) take what p holds
 * and add what it lacks.  The caller promises that the weight, bias and batch-norm arrays passed
 * with p are the same arrays with the same contents every time, until scn_params_clear(p) (after
 * an optimiser step, a load_state_dict) or scn_params_destroy(p); one object per convolution
 * module.  Results are bit-identical with and without.  No counterpart in the reference, whose
 * kernels read the weights as stored (CUDA/Convolution.cu:444-521). */
typedef struct scn_params scn_params;
scn_params *scn_params_create(void);
void scn_params_destroy(scn_params *p);
int scn_params_clear(scn_params *p);
int scn_md_use_params(scn_metadata *md, scn_params *p);

/* ActivePooling_updateOutput / ActivePooling_updateGradInput (pybind.cpp:34-43,
 * CPU/ActivePooling.cpp:8-83): out [batchSize, planes] = per sample the sum of its active rows, times
 * 1 / count when average != 0; d_in [nActive, planes] = the sample's gradient for each of its rows
 * (same factor).  The reference's rule builder (Metadata/ActivePoolingRules.h:16-34) does not return
 * for a sample with more than one site (its padding loop tests a constant); what is built here is the
 * rule matrix its header comment specifies, and agrees with the reference where that returns. */
int scn_active_pooling_fwd(scn_metadata *md, const int64_t *spatial, const float *in, float *out,
                           int planes, int average, void *stream);
int scn_active_pooling_bwd(scn_metadata *md, const int64_t *spatial, float *d_in, const float *d_out,
                           int planes, int average, void *stream);

/* ---- backward pass ----------------------------------------------------------------------------
 * Gradients are device fp32 arrays allocated by the caller and written in full (the reference's
 * Python side hands zero-filled tensors to calls that accumulate into them); d_bias may be NULL.
 * d_out is never modified. */

/* SubmanifoldConvolution_backward (pybind.cpp:140-146, CPU/Convolution.cpp:152-185):
 * d_in [nActive, nIn], d_weight as weight, d_bias [nOut] = column sums of d_out. */
int scn_subm_conv_bwd(scn_metadata *md, const int64_t *spatial, const int64_t *filter, const float *in,
                      float *d_in, const float *d_out, const float *weight, float *d_weight,
                      float *d_bias, int n_in, int n_out, int groups, void *stream);
/* Convolution_backward (pybind.cpp:61-66, CPU/Convolution.cpp:81-115). */
int scn_conv_bwd(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                 const int64_t *filter, const int64_t *stride, const float *in, float *d_in,
                 const float *d_out, const float *weight, float *d_weight, float *d_bias, int n_in,
                 int n_out, int groups, void *stream);
/* Deconvolution_backward (pybind.cpp:85-90, CPU/Deconvolution.cpp:43-77). */
int scn_deconv_bwd(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                   const int64_t *filter, const int64_t *stride, const float *in, float *d_in,
                   const float *d_out, const float *weight, float *d_weight, float *d_bias, int n_in,
                   int n_out, int groups, void *stream);
/* NetworkInNetwork_updateGradInput + NetworkInNetwork_accGradParameters (pybind.cpp:226-229,
 * CPU/NetworkInNetwork.cpp:24-47); the handle as for scn_nin_fwd. */
int scn_nin_bwd(scn_metadata *md, const float *in, float *d_in, const float *d_out, const float *weight,
                float *d_weight, float *d_bias, int64_t rows, int n_in, int n_out, void *stream);
/* BatchNormalization_updateOutput with train=true (pybind.cpp:220, CPU/BatchNormalization.cpp:13-61):
 * batch mean and 1/sqrt(biased variance + eps) into save_mean / save_invstd [planes]; running_mean /
 * running_var updated in place as momentum * old + (1 - momentum) * batch value (unbiased
 * variance); out = leaky(x * w + b) with the batch statistics.  The reference call takes no
 * metadata; here the handle owns the scratch of the column reductions (any handle will do; the
 * caller has the tensor's at hand).  rows == 0: save_mean and save_invstd are set to 0 and the
 * running statistics stay as they are (the reference divides by zero).  rows == 1: the unbiased
 * variance divides by rows - 1 = 0 and running_var becomes inf or nan, as in the reference. */
int scn_bn_train_fwd(scn_metadata *md, const float *in, float *out, int64_t rows, int planes,
                     int64_t in_stride, int64_t out_stride, float *save_mean, float *save_invstd,
                     float *running_mean, float *running_var, const float *gamma, const float *beta,
                     float eps, float momentum, float leakiness, void *stream);
/* BatchNormalization_backward (pybind.cpp:222, CPU/BatchNormalization.cpp:63-107,132-158), from
 * the statistics the forward pass saved.  d_gamma / d_beta may be NULL. */
int scn_bn_bwd(scn_metadata *md, const float *in, float *d_in, const float *out, const float *d_out,
               int64_t rows, int planes, int64_t in_stride, int64_t out_stride, const float *save_mean,
               const float *save_invstd, const float *gamma, float *d_gamma, float *d_beta,
               float leakiness, void *stream);
/* MaxPooling_updateGradInput (pybind.cpp:108-113, CPU/MaxPooling.cpp:21-35,61-87): d_in
 * [nActive(in_size), in_stride]; every input that equals its window's output receives that
 * window's gradient.  As in the reference, the comparison reads input planes [0, planes), without
 * the n_features_to_drop offset of the forward pass. */
int scn_maxpool_bwd(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                    const int64_t *size, const int64_t *stride, const float *in, float *d_in,
                    int in_stride, const float *out, const float *d_out, int planes,
                    int n_features_to_drop, void *stream);
/* AveragePooling_updateGradInput (pybind.cpp:49-54, CPU/AveragePooling.cpp:21-35,62-86). */
int scn_avgpool_bwd(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                    const int64_t *size, const int64_t *stride, float *d_in, int in_stride,
                    const float *d_out, int planes, int n_features_to_drop, void *stream);
/* UnPooling_updateGradInput (pybind.cpp:194-198, CPU/UnPooling.cpp:21-32,58-78): in_size is the
 * coarse level the unpooling's input lives on; d_in [nActive(in_size), in_stride]. */
int scn_unpool_bwd(scn_metadata *md, const int64_t *in_size, const int64_t *out_size,
                   const int64_t *size, const int64_t *stride, float *d_in, int in_stride,
                   const float *d_out, int planes, int n_features_to_drop, void *stream);
/* InputLayer_updateGradInput / BLInputLayer_updateGradInput (pybind.cpp:160-163,177-180,
 * CPU/IOLayers.cpp:73-93,161-184): d_out [nActive, planes] -> d_in [nInputRows, planes]. */
int scn_input_layer_bwd(scn_metadata *md, float *d_in, const float *d_out, int planes, void *stream);
/* OutputLayer_updateGradInput / BLOutputLayer_updateGradInput (pybind.cpp:168-171,185-188,
 * CPU/IOLayers.cpp:116-135,207-229): d_out [nInputRows, planes] -> d_in [nActive, planes]. */
int scn_output_layer_bwd(scn_metadata *md, float *d_in, const float *d_out, int planes, void *stream);
/* SparseToDense_updateGradInput (pybind.cpp:130-134, CPU/SparseToDense.cpp:21-33,66-90):
 * d_out [batch, planes, spatial...] -> d_in [nActive, planes]. */
int scn_s2d_bwd(scn_metadata *md, const int64_t *spatial, float *d_in, const float *d_out, int planes,
                void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SCN_HIP_H */
