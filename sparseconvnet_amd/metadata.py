"""Metadata: which sites are active at every spatial size, plus the cached rulebooks.

Mirrors the object the reference exposes as `sparseconvnet.Metadata(dim)`
(sparseconvnet/metadata.py:16-17 -> pybind class Metadata_<D>, SCN/pybind.cpp:11-33),
as a thin owner of a handle of libscn_hip.so.  Everything lives on the GPU; only counts
cross back to the host."""
import ctypes as C
import weakref

import torch

from . import _lib


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The caller's current stream as the library takes it.  Asked several times per module call:
    the raw handle costs a tenth of building a torch.cuda.Stream object around it."""
    if _raw_stream is not None:
        return C.c_void_p(_raw_stream(torch.cuda.current_device()))
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None and t.numel() else C.c_void_p(0)


def _mark_written(t):
    """Moves the version counter of a tensor the library has written to behind torch's back."""
    try:
        torch.autograd.graph.increment_version(t)
    except AttributeError:  # older torch: drop everything that is keyed on version counters instead
        import sparseconvnet_amd
        sparseconvnet_amd.parameters_changed()


def _features(t, what):
    if not t.is_cuda:
        raise _lib.ScnError("%s must be a CUDA tensor: this library has no CPU path" % what)
    if t.dtype != torch.float32:
        raise _lib.ScnError("%s must be float32" % what)
    return t.contiguous()


class MacCounter:
    """The package's forward_pass_multiplyAdd_count (sparseconvnet/__init__.py:7).  The
    convolutions do not fetch their rule counts when they run (that would stall the GPU once
    per rulebook); the library keeps a running total per Metadata, which is collected here
    when somebody reads the counter or the Metadata goes away."""

    def __init__(self):
        self.base = 0.0
        self.live = weakref.WeakSet()

    def _released(self):
        """What Metadata objects that are gone still owed (the library settles those counts
        without stalling when a Metadata dies; this waits for them)."""
        macs = C.c_double(0)
        _lib.check(_lib.lib().scn_take_released_macs(C.byref(macs)))
        return macs.value

    def read(self):
        for md in list(self.live):
            self.base += md.takeMacs()
        self.base += self._released()
        return self.base

    def reset(self, value):
        for md in list(self.live):
            md.takeMacs()
        self._released()
        self.base = value


mac_counter = MacCounter()


class Metadata:
    def __init__(self, dimension):
        self.dimension = dimension
        self._L = _lib.lib()
        self._h = self._L.scn_md_create(dimension)
        if not self._h:
            raise _lib.ScnError(self._L.scn_last_error().decode())
        mac_counter.live.add(self)
        import sparseconvnet_amd
        if getattr(sparseconvnet_amd, "bf16_mfma", False):
            self.setBf16(True)

    def setBf16(self, enable):
        """Wide convolutions of this Metadata round their operands to bf16 and accumulate in
        fp32 (about 1e-2 relative to the output scale); everything else stays fp32."""
        _lib.check(self._L.scn_md_set_bf16(self._h, 1 if enable else 0))

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            self._h = None
            self._L.scn_md_destroy(h)  # does not wait for the GPU; the counts it owes are kept (MacCounter)

    def takeMacs(self):
        """Multiply-adds of the convolutions run on this Metadata since the last call whose
        count was not returned to the caller directly (synchronises the stream once)."""
        macs = C.c_double(0)
        _lib.check(self._L.scn_md_take_macs(self._h, _stream(), C.byref(macs)))
        return macs.value

    def _s(self, x):
        return _lib.sizes(self.dimension, x)

    # ---- what the reference binds on Metadata_<D> ------------------------------------
    def clear(self):
        _lib.check(self._L.scn_md_clear(self._h))

    def getNActive(self, spatial_size):
        n = C.c_int64(0)
        _lib.check(self._L.scn_md_nactive(self._h, self._s(spatial_size), C.byref(n)))
        return n.value

    def getBatchSize(self, spatial_size):
        b = C.c_int(0)
        _lib.check(self._L.scn_md_batch_size(self._h, self._s(spatial_size), C.byref(b)))
        return b.value

    def getSpatialLocations(self, spatial_size):
        """LongTensor [nActive, dimension+1] on the CPU: coordinates, then sample index."""
        n = self.getNActive(spatial_size)
        out = torch.zeros((n, self.dimension + 1), dtype=torch.int64, device="cuda")
        if n:
            _lib.check(self._L.scn_md_spatial_locations(self._h, self._s(spatial_size), _ptr(out), _stream()))
        return out.cpu()

    # ---- forward ops; each returns a new CUDA tensor ---------------------------------
    def inputLayer(self, spatial_size, coords, features, batch_size, mode):
        assert coords.dim() == 2 and coords.size(0) == features.size(0)
        features = _features(features, "input features")
        n = C.c_int64(0)
        if coords.device.type == "cpu":
            # the reference's calling convention (ioLayers.py:51-65): the library reads the host
            # tensor itself, narrowing the values on their way to the device
            coords = coords.to(dtype=torch.int64).contiguous()
            _lib.check(self._L.scn_md_input_layer_host(self._h, self._s(spatial_size), C.c_void_p(coords.data_ptr()),
                                                       coords.size(0), coords.size(1), int(batch_size), int(mode),
                                                       _stream(), C.byref(n)))
        else:
            coords = coords.to(device=features.device, dtype=torch.int64).contiguous()
            _lib.check(self._L.scn_md_input_layer(self._h, self._s(spatial_size), _ptr(coords), coords.size(0),
                                                  coords.size(1), int(batch_size), int(mode), _stream(),
                                                  C.byref(n)))
        out = torch.empty((n.value, features.size(1)), dtype=torch.float32, device=features.device)
        _lib.check(self._L.scn_input_layer_fwd(self._h, _ptr(features), _ptr(out), features.size(1), _stream()))
        return out

    def inputBatch(self, spatial_size, coords, vectors, overwrite, batch_size):
        """Everything an InputBatch collected, in the order it was set: coords [n, dimension
        (+1)], vectors [n, planes], overwrite None or a uint8 tensor [n] (points that replace
        what their site holds) -> features [nActive, planes], rows by first occurrence."""
        coords = coords.to(device=vectors.device, dtype=torch.int64).contiguous()
        assert coords.dim() == 2 and coords.size(0) == vectors.size(0)
        vectors = _features(vectors, "input vectors")
        if overwrite is not None:
            overwrite = overwrite.to(device=vectors.device, dtype=torch.uint8).contiguous()
            assert overwrite.numel() == coords.size(0)
        n = C.c_int64(0)
        _lib.check(self._L.scn_md_input_batch(self._h, self._s(spatial_size), _ptr(coords), _ptr(overwrite),
                                              coords.size(0), coords.size(1), int(batch_size), _stream(),
                                              C.byref(n)))
        out = torch.empty((n.value, vectors.size(1)), dtype=torch.float32, device=vectors.device)
        _lib.check(self._L.scn_input_layer_fwd(self._h, _ptr(vectors), _ptr(out), vectors.size(1), _stream()))
        return out

    def generateRuleBooks2s2(self):
        """3^d submanifold and 2^d / stride-2 rulebooks of every level, ahead of their use."""
        _lib.check(self._L.scn_md_generate_rulebooks(self._h, 2, _stream()))

    def generateRuleBooks3s2(self):
        """3^d submanifold and 3^d / stride-2 rulebooks of every level, ahead of their use."""
        _lib.check(self._L.scn_md_generate_rulebooks(self._h, 3, _stream()))

    def outputLayer(self, features):
        features = _features(features, "features")
        hdr = (C.c_int32 * 4)()
        _lib.check(self._L.scn_md_input_rules_header(self._h, hdr))
        out = torch.empty((hdr[2], features.size(1)), dtype=torch.float32, device=features.device)
        _lib.check(self._L.scn_output_layer_fwd(self._h, _ptr(features), _ptr(out), features.size(1), _stream()))
        return out

    def blInputLayer(self, spatial_size, coords, features, mode):
        """coords [batch, length, dimension] (first coordinate < 0: empty position),
        features [batch, length, planes] -> [nActive, planes]."""
        coords = coords.to(device=features.device, dtype=torch.int64).contiguous()
        assert coords.dim() == 3 and features.dim() == 3 and coords.shape[:2] == features.shape[:2], \
            (coords.shape, features.shape)
        features = _features(features, "input features")
        n = C.c_int64(0)
        _lib.check(self._L.scn_md_bl_input_layer(self._h, self._s(spatial_size), _ptr(coords), coords.size(0),
                                                 coords.size(1), int(mode), _stream(), C.byref(n)))
        out = torch.empty((n.value, features.size(2)), dtype=torch.float32, device=features.device)
        _lib.check(self._L.scn_input_layer_fwd(self._h, _ptr(features), _ptr(out), features.size(2), _stream()))
        return out

    def blOutputLayer(self, features):
        """[nActive, planes] -> [batch, length, planes] of the batch-by-length input layer."""
        features = _features(features, "features")
        hdr = (C.c_int32 * 5)()
        _lib.check(self._L.scn_md_bl_rules_header(self._h, hdr))
        out = torch.empty((hdr[2], hdr[3], features.size(1)), dtype=torch.float32, device=features.device)
        _lib.check(self._L.scn_output_layer_fwd(self._h, _ptr(features), _ptr(out), features.size(1), _stream()))
        return out

    def _conv(self, kind, size_args, n_rows, features, weight, bias, bn, post, want_macs, out=None, second=None):
        """kind 0 / 1 / 2: submanifold / strided / transposed convolution.  bn, post: None, or
        (running_mean, running_var, weight, bias, eps, leakiness) of an eval-mode batch
        normalisation in front of / behind the convolution, applied inside it.  want_macs:
        return the multiply-add count (a stream synchronisation the first time a rulebook is
        used); otherwise the library adds it to this Metadata's running total (takeMacs).
        out: a [rows, planes] range of columns of a wider float32 matrix to write the result into
        (the convolution's part of a concatenation), or None for a new tensor.
        second: None, or (batch norm arguments, columns as for `out`): the convolution also writes
        its output there, taken before `post` and normalised with that batch norm instead."""
        features = _features(features, "features")
        weight = _features(weight, "weight")
        K, groups, ip, op = weight.shape
        bias_t = _features(bias, "bias") if bias is not None and bias.numel() else None
        resets = []  # what serves this one call is taken back, also when the call fails before it gets there
        try:
            if second is not None and n_rows:
                bn2, out2 = second
                assert out2.dtype == torch.float32 and out2.device == features.device and out2.dim() == 2, out2
                assert tuple(out2.shape) == (n_rows, groups * op) and out2.stride(1) == 1, (out2.shape, out2.stride())
                mean, var, g, b, eps, leak = bn2
                t = [_features(mean, "running_mean"), _features(var, "running_var"),
                     _features(g, "bn weight") if g is not None and g.numel() else None,
                     _features(b, "bn bias") if b is not None and b.numel() else None]
                resets.append(lambda: self._L.scn_md_next_second_output(self._h, None, 0, None))
                _lib.check(self._L.scn_md_next_second_output(
                    self._h, _ptr(out2), out2.stride(0),
                    C.byref(_lib.BnParams(*[_ptr(x) for x in t], float(eps), float(leak)))))
            if out is None:
                out = torch.empty((n_rows, groups * op), dtype=torch.float32, device=features.device)
            else:
                assert out.dtype == torch.float32 and out.device == features.device and out.dim() == 2, out
                assert tuple(out.shape) == (n_rows, groups * op) and out.stride(1) == 1, (out.shape, out.stride())
                if n_rows and out.stride(0) != out.size(1):
                    resets.append(lambda: self._L.scn_md_next_output_stride(self._h, 0))
                    _lib.check(self._L.scn_md_next_output_stride(self._h, out.stride(0)))
            return self._conv_into(kind, size_args, features, weight, bias_t, bn, post, want_macs, out)
        finally:
            for r in resets:
                r()

    def _conv_into(self, kind, size_args, features, weight, bias_t, bn, post, want_macs, out):
        K, groups, ip, op = weight.shape
        macs = C.c_double(0)
        macs_p = C.byref(macs) if want_macs else None
        tail = (_ptr(features), _ptr(out), _ptr(weight), _ptr(bias_t), groups * ip, groups * op, groups)
        if bn is None and post is None:
            fn = (self._L.scn_subm_conv_fwd, self._L.scn_conv_fwd, self._L.scn_deconv_fwd)[kind]
            _lib.check(fn(self._h, *size_args, *tail, _stream(), macs_p))
        else:
            keep = []  # tensors behind the raw pointers stay alive until the call has been issued

            def params(p, planes):
                if p is None:
                    return None
                mean, var, g, b, eps, leak = p
                assert mean.numel() == planes and var.numel() == planes, (mean.shape, planes)
                t = [_features(mean, "running_mean"), _features(var, "running_var"),
                     _features(g, "bn weight") if g is not None and g.numel() else None,
                     _features(b, "bn bias") if b is not None and b.numel() else None]
                keep.extend(t)
                return C.byref(_lib.BnParams(*[_ptr(x) for x in t], float(eps), float(leak)))
            sizes = list(size_args) + [None] * (4 - len(size_args))
            _lib.check(self._L.scn_conv_bn_fwd(self._h, kind, *sizes, *tail, params(bn, groups * ip),
                                               params(post, groups * op), _stream(), macs_p))
        return out, (macs.value if want_macs else None)

    def submanifoldConvolution(self, spatial_size, filter_size, features, weight, bias, bn=None, post=None,
                               want_macs=True, out=None, second=None):
        sp, fs = self._s(spatial_size), self._s(filter_size)
        _lib.check(self._L.scn_md_submanifold_rules(self._h, sp, fs, _stream()))
        return self._conv(0, (sp, fs), self.getNActive(spatial_size), features, weight, bias, bn, post, want_macs, out, second)

    def convolution(self, in_size, out_size, filter_size, stride, features, weight, bias, bn=None, post=None,
                    want_macs=True, out=None, second=None):
        a = [self._s(v) for v in (in_size, out_size, filter_size, stride)]
        _lib.check(self._L.scn_md_strided_rules(self._h, *a, _stream()))
        return self._conv(1, a, self.getNActive(out_size), features, weight, bias, bn, post, want_macs, out, second)

    def deconvolution(self, in_size, out_size, filter_size, stride, features, weight, bias, bn=None, post=None,
                      want_macs=True, out=None, second=None):
        a = [self._s(v) for v in (in_size, out_size, filter_size, stride)]
        rb = [self._s(v) for v in (out_size, in_size, filter_size, stride)]
        _lib.check(self._L.scn_md_strided_rules(self._h, *rb, _stream()))
        return self._conv(2, a, self.getNActive(out_size), features, weight, bias, bn, post, want_macs, out, second)

    def networkInNetwork(self, features, weight, bias, want_macs=True):
        """out = bias + features @ weight (weight [nIn, nOut]): a convolution with one tap."""
        features = _features(features, "features")
        weight = _features(weight, "weight")
        bias_t = _features(bias, "bias") if bias is not None and bias.numel() else None
        n_in, n_out = weight.shape
        assert features.size(0) == 0 or features.size(1) == n_in, (features.shape, weight.shape)
        out = torch.empty((features.size(0), n_out), dtype=torch.float32, device=features.device)
        macs = C.c_double(0)
        _lib.check(self._L.scn_nin_fwd(self._h, _ptr(features), _ptr(out), _ptr(weight), _ptr(bias_t),
                                       features.size(0), n_in, n_out, _stream(),
                                       C.byref(macs) if want_macs else None))
        return out, (macs.value if want_macs else None)

    def _pool(self, fn, rule_sizes, a, n_rows, features, n_features_to_drop):
        _lib.check(self._L.scn_md_strided_rules(self._h, *rule_sizes, _stream()))
        features = _features(features, "features")
        planes = features.size(1) - n_features_to_drop
        out = torch.empty((n_rows(), planes), dtype=torch.float32, device=features.device)
        _lib.check(fn(self._h, *a, _ptr(features), features.size(1), _ptr(out), planes, n_features_to_drop,
                      _stream()))
        return out

    def maxPooling(self, in_size, out_size, pool_size, pool_stride, features, n_features_to_drop):
        a = [self._s(v) for v in (in_size, out_size, pool_size, pool_stride)]
        return self._pool(self._L.scn_maxpool_fwd, a, a, lambda: self.getNActive(out_size), features,
                          n_features_to_drop)

    def averagePooling(self, in_size, out_size, pool_size, pool_stride, features, n_features_to_drop):
        a = [self._s(v) for v in (in_size, out_size, pool_size, pool_stride)]
        return self._pool(self._L.scn_avgpool_fwd, a, a, lambda: self.getNActive(out_size), features,
                          n_features_to_drop)

    def unPooling(self, in_size, out_size, pool_size, pool_stride, features, n_features_to_drop):
        """in_size: the coarse level the features live on; out_size: the finer level."""
        a = [self._s(v) for v in (in_size, out_size, pool_size, pool_stride)]
        rb = [self._s(v) for v in (out_size, in_size, pool_size, pool_stride)]
        return self._pool(self._L.scn_unpool_fwd, rb, a, lambda: self.getNActive(out_size), features,
                          n_features_to_drop)

    def sparseToDense(self, spatial_size, features, n_planes):
        features = _features(features, "features")
        sp = [int(v) for v in self._s(spatial_size)]
        out = torch.empty([self.getBatchSize(spatial_size), n_planes] + sp, dtype=torch.float32,
                          device=features.device)
        _lib.check(self._L.scn_s2d_fwd(self._h, self._s(spatial_size), _ptr(features), _ptr(out), n_planes,
                                       _stream()))
        return out

    def activePooling(self, spatial_size, features, average):
        """ActivePooling_updateOutput (pybind.cpp:34-38): [batchSize, planes], per sample the sum
        (average: the mean) of its active rows."""
        features = _features(features, "features")
        out = torch.empty((self.getBatchSize(spatial_size), features.size(1)), dtype=torch.float32,
                          device=features.device)
        _lib.check(self._L.scn_active_pooling_fwd(self._h, self._s(spatial_size), _ptr(features), _ptr(out),
                                                  features.size(1), int(bool(average)), _stream()))
        return out

    def activePoolingBackward(self, spatial_size, shape, grad_output, average):
        """ActivePooling_updateGradInput (pybind.cpp:39-43): shape = that of the op's input."""
        grad_output = _features(grad_output, "grad_output")
        d_in = torch.empty(shape, dtype=torch.float32, device=grad_output.device)
        if d_in.numel():
            _lib.check(self._L.scn_active_pooling_bwd(self._h, self._s(spatial_size), _ptr(d_in), _ptr(grad_output),
                                                      shape[1], int(bool(average)), _stream()))
        return d_in

    # ---- backward ops: each returns the gradients the reference's backward call fills ----------
    def _convBackward(self, fn, size_args, features, grad_output, weight, with_bias):
        features = _features(features, "features")
        grad_output = _features(grad_output, "grad_output")
        weight = _features(weight, "weight")
        K, groups, ip, op = weight.shape
        d_in = torch.empty_like(features)
        d_w = torch.empty_like(weight)
        d_b = torch.empty((groups * op,), dtype=torch.float32, device=features.device) if with_bias else None
        _lib.check(fn(self._h, *size_args, _ptr(features), _ptr(d_in), _ptr(grad_output), _ptr(weight), _ptr(d_w),
                      _ptr(d_b), groups * ip, groups * op, groups, _stream()))
        return d_in, d_w, d_b

    def submanifoldConvolutionBackward(self, spatial_size, filter_size, features, grad_output, weight, with_bias):
        return self._convBackward(self._L.scn_subm_conv_bwd, (self._s(spatial_size), self._s(filter_size)), features,
                                  grad_output, weight, with_bias)

    def convolutionBackward(self, in_size, out_size, filter_size, stride, features, grad_output, weight, with_bias):
        a = [self._s(v) for v in (in_size, out_size, filter_size, stride)]
        return self._convBackward(self._L.scn_conv_bwd, a, features, grad_output, weight, with_bias)

    def deconvolutionBackward(self, in_size, out_size, filter_size, stride, features, grad_output, weight, with_bias):
        a = [self._s(v) for v in (in_size, out_size, filter_size, stride)]
        return self._convBackward(self._L.scn_deconv_bwd, a, features, grad_output, weight, with_bias)

    def networkInNetworkBackward(self, features, grad_output, weight, with_bias):
        features = _features(features, "features")
        grad_output = _features(grad_output, "grad_output")
        weight = _features(weight, "weight")
        n_in, n_out = weight.shape
        d_in, d_w = torch.empty_like(features), torch.empty_like(weight)
        d_b = torch.empty((n_out,), dtype=torch.float32, device=features.device) if with_bias else None
        _lib.check(self._L.scn_nin_bwd(self._h, _ptr(features), _ptr(d_in), _ptr(grad_output), _ptr(weight), _ptr(d_w),
                                       _ptr(d_b), features.size(0), n_in, n_out, _stream()))
        return d_in, d_w, d_b

    def batchNormTrain(self, features, running_mean, running_var, weight, bias, eps, momentum, leakiness):
        """Training-mode forward: (output, saved mean, saved 1/std); running statistics updated in place."""
        features = _features(features, "features")
        out = torch.empty_like(features)
        planes = features.size(1)
        save_mean = torch.empty(planes, dtype=torch.float32, device=features.device)
        save_invstd = torch.empty(planes, dtype=torch.float32, device=features.device)
        w = weight if weight is not None and weight.numel() else None
        b = bias if bias is not None and bias.numel() else None
        _lib.check(self._L.scn_bn_train_fwd(self._h, _ptr(features), _ptr(out), features.size(0), planes,
                                            features.stride(0), out.stride(0), _ptr(save_mean), _ptr(save_invstd),
                                            _ptr(running_mean), _ptr(running_var), _ptr(w), _ptr(b), float(eps),
                                            float(momentum), float(leakiness), _stream()))
        # The library wrote the running statistics through raw pointers: tell torch, so that whatever is
        # keyed on their version counters (the folded batch norms eval-mode convolutions keep) notices.
        for t in (running_mean, running_var):
            if t is not None:
                _mark_written(t)
        return out, save_mean, save_invstd

    def batchNormBackward(self, features, output, grad_output, save_mean, save_invstd, weight, leakiness, affine):
        features = _features(features, "features")
        grad_output = _features(grad_output, "grad_output")
        planes = features.size(1)
        d_in = torch.empty_like(features)
        d_w = torch.empty(planes, dtype=torch.float32, device=features.device) if affine else None
        d_b = torch.empty(planes, dtype=torch.float32, device=features.device) if affine else None
        w = weight if weight is not None and weight.numel() else None
        _lib.check(self._L.scn_bn_bwd(self._h, _ptr(features), _ptr(d_in), _ptr(output), _ptr(grad_output),
                                      features.size(0), planes, features.stride(0), output.stride(0), _ptr(save_mean),
                                      _ptr(save_invstd), _ptr(w), _ptr(d_w), _ptr(d_b), float(leakiness), _stream()))
        return d_in, d_w, d_b

    def maxPoolingBackward(self, in_size, out_size, pool_size, pool_stride, features, output, grad_output,
                           n_features_to_drop):
        a = [self._s(v) for v in (in_size, out_size, pool_size, pool_stride)]
        features = _features(features, "features")
        grad_output = _features(grad_output, "grad_output")
        d_in = torch.empty_like(features)
        if features.size(0):
            _lib.check(self._L.scn_maxpool_bwd(self._h, *a, _ptr(features), _ptr(d_in), features.size(1), _ptr(output),
                                               _ptr(grad_output), output.size(1), n_features_to_drop, _stream()))
        return d_in

    def averagePoolingBackward(self, in_size, out_size, pool_size, pool_stride, input_shape, grad_output,
                               n_features_to_drop):
        a = [self._s(v) for v in (in_size, out_size, pool_size, pool_stride)]
        grad_output = _features(grad_output, "grad_output")
        d_in = torch.empty(tuple(input_shape), dtype=torch.float32, device=grad_output.device)
        if d_in.size(0):
            _lib.check(self._L.scn_avgpool_bwd(self._h, *a, _ptr(d_in), d_in.size(1), _ptr(grad_output),
                                               grad_output.size(1), n_features_to_drop, _stream()))
        return d_in

    def unPoolingBackward(self, in_size, out_size, pool_size, pool_stride, input_shape, grad_output,
                          n_features_to_drop):
        a = [self._s(v) for v in (in_size, out_size, pool_size, pool_stride)]
        grad_output = _features(grad_output, "grad_output")
        d_in = torch.empty(tuple(input_shape), dtype=torch.float32, device=grad_output.device)
        if d_in.size(0):
            _lib.check(self._L.scn_unpool_bwd(self._h, *a, _ptr(d_in), d_in.size(1), _ptr(grad_output),
                                              grad_output.size(1), n_features_to_drop, _stream()))
        return d_in

    def inputLayerBackward(self, grad_output, bl=False):
        """d(features of the points) from d(features of the sites); bl: [batch, length, planes]."""
        grad_output = _features(grad_output, "grad_output")
        planes = grad_output.size(1)
        if bl:
            hdr = (C.c_int32 * 5)()
            _lib.check(self._L.scn_md_bl_rules_header(self._h, hdr))
            d_in = torch.empty((hdr[2], hdr[3], planes), dtype=torch.float32, device=grad_output.device)
        else:
            hdr = (C.c_int32 * 4)()
            _lib.check(self._L.scn_md_input_rules_header(self._h, hdr))
            d_in = torch.empty((hdr[2], planes), dtype=torch.float32, device=grad_output.device)
        if d_in.numel():
            _lib.check(self._L.scn_input_layer_bwd(self._h, _ptr(d_in), _ptr(grad_output), planes, _stream()))
        return d_in

    def outputLayerBackward(self, grad_output, n_active):
        """d(features of the sites) from d(features of the points) ([points, planes] or [batch, length, planes])."""
        grad_output = _features(grad_output, "grad_output")
        planes = grad_output.size(-1)
        d_in = torch.empty((n_active, planes), dtype=torch.float32, device=grad_output.device)
        if d_in.numel():
            _lib.check(self._L.scn_output_layer_bwd(self._h, _ptr(d_in), _ptr(grad_output), planes, _stream()))
        return d_in

    def sparseToDenseBackward(self, spatial_size, grad_output, n_active):
        grad_output = _features(grad_output, "grad_output")
        d_in = torch.empty((n_active, grad_output.size(1)), dtype=torch.float32, device=grad_output.device)
        if d_in.numel():
            _lib.check(self._L.scn_s2d_bwd(self._h, self._s(spatial_size), _ptr(d_in), _ptr(grad_output),
                                           grad_output.size(1), _stream()))
        return d_in


def batchNormEval(features, running_mean, running_var, weight, bias, eps, leakiness, out=None):
    """out: where the result goes, rows of features.size(1) floats at any row stride (a column
    range of a wider matrix); a new tensor when None."""
    features = _features(features, "features")
    if out is None:
        out = torch.empty_like(features)
    assert out.shape == features.shape and out.stride(1) == 1 and out.dtype == torch.float32 and out.is_cuda
    w = weight if weight is not None and weight.numel() else None
    b = bias if bias is not None and bias.numel() else None
    _lib.check(_lib.lib().scn_bn_eval_fwd(_ptr(features), _ptr(out), features.size(0), features.size(1),
                                          features.stride(0), out.stride(0), _ptr(running_mean),
                                          _ptr(running_var), _ptr(w), _ptr(b), float(eps), float(leakiness),
                                          _stream()))
    return out
