"""ctypes driver for the CPU checkers (TEST INFRASTRUCTURE ONLY).

`CpuPath("oracle")` drives oracle/libscn_oracle.so, this repository's own CPU
restatement of the reference algorithm; `CpuPath("ref")` drives
oracle/_ref/libscn_ref.so, the reference's CPU sources compiled behind
oracle/ref_harness.cpp (present only where oracle/Makefile could build it).
Both expose the same entry points, so one class serves both.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; the shipped package never does.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATHS = {"oracle": os.path.join(_HERE, "libscn_oracle.so"),
          "ref": os.path.join(_HERE, "_ref", "libscn_ref.so")}
_PREFIX = {"oracle": "orc_", "ref": "ref_"}
_libs = {}

_i64p = C.POINTER(C.c_int64)
_i32p = C.POINTER(C.c_int32)
_f32p = C.POINTER(C.c_float)


def available(flavour):
    return os.path.exists(_PATHS[flavour])


def _load(flavour):
    if flavour in _libs:
        return _libs[flavour]
    if flavour == "ref":
        import torch  # noqa: F401  (libscn_ref.so links libtorch_cpu)
    lib = C.CDLL(_PATHS[flavour])
    p = _PREFIX[flavour]
    sig = {
        "md_create": (C.c_void_p, [C.c_int]),
        "md_destroy": (None, [C.c_void_p]),
        "input_layer": (C.c_int, [C.c_void_p, _i64p, _i64p, C.c_int, C.c_int, C.c_int, C.c_int]),
        "input_rules_header": (None, [C.c_void_p, _i32p]),
        "input_rules": (None, [C.c_void_p, _i32p]),
        "bl_input_layer": (C.c_int, [C.c_void_p, _i64p, _i64p, C.c_int, C.c_int, C.c_int]),
        "bl_rules_header": (None, [C.c_void_p, _i32p]),
        "bl_rules": (None, [C.c_void_p, _i32p]),
        "bl_input_fwd": (None, [C.c_void_p, _f32p, _f32p, C.c_int]),
        "bl_output_fwd": (None, [C.c_void_p, _f32p, _f32p, C.c_int]),
        "set_input_spatial_size": (None, [C.c_void_p, _i64p]),
        "batch_add_sample": (None, [C.c_void_p]),
        "set_input_locations": (C.c_int, [C.c_void_p, _i64p, C.c_int, C.c_int, _f32p, C.c_int, C.c_int]),
        "add_sample_from_tensor": (None, [C.c_void_p, _f32p, _i64p, C.c_int, _i64p, C.c_float]),
        "batch_planes": (C.c_int, [C.c_void_p]),
        "batch_features": (None, [C.c_void_p, _f32p]),
        "generate_rulebooks": (None, [C.c_void_p, C.c_int]),
        "nactive": (C.c_int, [C.c_void_p, _i64p]),
        "batch_size": (C.c_int, [C.c_void_p, _i64p]),
        "spatial_locations": (None, [C.c_void_p, _i64p, _i64p]),
        "rb_noffsets": (C.c_int, [C.c_void_p, C.c_int, _i64p, _i64p, _i64p, _i64p]),
        "rb_counts": (None, [C.c_void_p, C.c_int, _i64p, _i64p, _i64p, _i64p, _i64p]),
        "rb_copy": (None, [C.c_void_p, C.c_int, _i64p, _i64p, _i64p, _i64p, C.c_int, _i32p]),
        "subm_conv": (C.c_double, [C.c_void_p, _i64p, _i64p, _f32p, _f32p, _f32p, _f32p,
                                   C.c_int, C.c_int, C.c_int]),
        "conv": (C.c_double, [C.c_void_p, _i64p, _i64p, _i64p, _i64p, _f32p, _f32p, _f32p, _f32p,
                              C.c_int, C.c_int, C.c_int]),
        "deconv": (C.c_double, [C.c_void_p, _i64p, _i64p, _i64p, _i64p, _f32p, _f32p, _f32p,
                                _f32p, C.c_int, C.c_int, C.c_int]),
        "maxpool": (None, [C.c_void_p, _i64p, _i64p, _i64p, _i64p, _f32p, C.c_int, _f32p,
                           C.c_int, C.c_int]),
        "avgpool": (None, [C.c_void_p, _i64p, _i64p, _i64p, _i64p, _f32p, C.c_int, _f32p,
                           C.c_int, C.c_int]),
        "unpool": (None, [C.c_void_p, _i64p, _i64p, _i64p, _i64p, _f32p, C.c_int, _f32p,
                          C.c_int, C.c_int]),
        "nin": (C.c_double, [_f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]),
        "bn_eval": (None, [_f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _f32p, _f32p,
                           _f32p, C.c_float, C.c_float]),
        "input_fwd": (None, [C.c_void_p, _f32p, _f32p, C.c_int]),
        "output_fwd": (None, [C.c_void_p, _f32p, _f32p, C.c_int]),
        "s2d": (None, [C.c_void_p, _i64p, _f32p, _f32p, C.c_int]),
        # backward pass
        "subm_conv_bwd": (None, [C.c_void_p, _i64p, _i64p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p,
                                 C.c_int, C.c_int, C.c_int]),
        "conv_bwd": (None, [C.c_void_p, _i64p, _i64p, _i64p, _i64p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p,
                            C.c_int, C.c_int, C.c_int]),
        "deconv_bwd": (None, [C.c_void_p, _i64p, _i64p, _i64p, _i64p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p,
                              C.c_int, C.c_int, C.c_int]),
        "nin_bwd": (None, [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]),
        "bn_train": (None, [_f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _f32p, _f32p, _f32p, _f32p,
                            _f32p, C.c_float, C.c_float, C.c_float]),
        "bn_bwd": (None, [_f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _f32p, _f32p,
                          _f32p, _f32p, C.c_float]),
        "maxpool_bwd": (None, [C.c_void_p, _i64p, _i64p, _i64p, _i64p, _f32p, _f32p, C.c_int, _f32p, _f32p,
                               C.c_int, C.c_int]),
        "avgpool_bwd": (None, [C.c_void_p, _i64p, _i64p, _i64p, _i64p, _f32p, C.c_int, _f32p, C.c_int, C.c_int]),
        "unpool_bwd": (None, [C.c_void_p, _i64p, _i64p, _i64p, _i64p, _f32p, C.c_int, _f32p, C.c_int, C.c_int]),
        "input_bwd": (None, [C.c_void_p, _f32p, _f32p, C.c_int]),
        "output_bwd": (None, [C.c_void_p, _f32p, _f32p, C.c_int]),
        "bl_input_bwd": (None, [C.c_void_p, _f32p, _f32p, C.c_int]),
        "bl_output_bwd": (None, [C.c_void_p, _f32p, _f32p, C.c_int]),
        "s2d_bwd": (None, [C.c_void_p, _i64p, _f32p, _f32p, C.c_int]),
        "active_pooling": (C.c_int, [C.c_void_p, _i64p, _f32p, _f32p, C.c_int, C.c_int]),
        "active_pooling_bwd": (C.c_int, [C.c_void_p, _i64p, _f32p, _f32p, C.c_int, C.c_int]),
    }
    fns = {}
    for name, (res, args) in sig.items():
        f = getattr(lib, p + name)
        f.restype = res
        f.argtypes = args
        fns[name] = f
    _libs[flavour] = fns
    return fns


def _sz(dim, x):
    a = np.ascontiguousarray(np.broadcast_to(np.asarray(x, dtype=np.int64), (dim,)))
    return a


def _p64(a):
    return a.ctypes.data_as(_i64p) if a is not None else None


def _pf(a):
    return a.ctypes.data_as(_f32p) if a is not None else None


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


class CpuPath:
    """One Metadata object of the CPU path plus the forward and backward ops that use it."""

    def __init__(self, dim, flavour="oracle"):
        self.f = _load(flavour)
        self.dim = dim
        self.h = self.f["md_create"](dim)
        if not self.h:
            raise ValueError("unsupported dimension %d" % dim)

    def __del__(self):
        if getattr(self, "h", None):
            self.f["md_destroy"](self.h)
            self.h = None

    # -- metadata ---------------------------------------------------------
    def input_layer(self, spatial, coords, batch_size=0, mode=3):
        coords = np.ascontiguousarray(coords, dtype=np.int64)
        s = _sz(self.dim, spatial)
        self.input_spatial = s
        return self.f["input_layer"](self.h, _p64(s), _p64(coords), coords.shape[0],
                                     coords.shape[1], batch_size, mode)

    def input_rules(self):
        hdr = np.zeros(4, np.int32)
        self.f["input_rules_header"](self.h, hdr.ctypes.data_as(_i32p))
        mode, max_active, n_in, n_out = [int(v) for v in hdr]
        rows = np.zeros((n_out, 1 + max_active), np.int32)
        if mode != 0 and n_out:
            self.f["input_rules"](self.h, rows.ctypes.data_as(_i32p))
        return hdr, rows

    # batch-by-length input layer: coords [batch, length, dim], features [batch, length, planes]
    def bl_input_layer(self, spatial, coords, mode=3):
        coords = np.ascontiguousarray(coords, dtype=np.int64)
        assert coords.ndim == 3 and coords.shape[2] == self.dim
        return self.f["bl_input_layer"](self.h, _p64(_sz(self.dim, spatial)), _p64(coords),
                                        coords.shape[0], coords.shape[1], mode)

    def bl_rules(self):
        """(header [mode, maxActive, batch, length, nOut], rows [nOut, 1 + maxActive])."""
        hdr = np.zeros(5, np.int32)
        self.f["bl_rules_header"](self.h, hdr.ctypes.data_as(_i32p))
        rows = np.zeros((int(hdr[4]), 1 + int(hdr[1])), np.int32)
        if hdr[0] != 0 and hdr[4]:
            self.f["bl_rules"](self.h, rows.ctypes.data_as(_i32p))
        return hdr, rows

    def bl_input_fwd(self, x):
        x = _f32(x)
        hdr, _ = self.bl_rules()
        flat = np.ascontiguousarray(x.reshape(-1, x.shape[-1]))
        out = np.zeros((int(hdr[4]), x.shape[-1]), np.float32)
        self.f["bl_input_fwd"](self.h, _pf(flat), _pf(out), x.shape[-1])
        return out

    def bl_output_fwd(self, x):
        x = _f32(x)
        hdr, _ = self.bl_rules()
        out = np.zeros((int(hdr[2]), int(hdr[3]), x.shape[1]), np.float32)
        self.f["bl_output_fwd"](self.h, _pf(x), _pf(out), x.shape[1])
        return out

    # point-at-a-time input (sparseconvnet/inputBatch.py)
    def batch_begin(self, spatial):
        self.input_spatial = _sz(self.dim, spatial)
        self.f["set_input_spatial_size"](self.h, _p64(self.input_spatial))

    def batch_add_sample(self):
        self.f["batch_add_sample"](self.h)

    def batch_set_locations(self, locations, vectors, overwrite=False):
        locations = np.ascontiguousarray(locations, dtype=np.int64)
        vectors = _f32(vectors)
        assert locations.ndim == 2 and vectors.ndim == 2 and len(locations) == len(vectors)
        r = self.f["set_input_locations"](self.h, _p64(locations), locations.shape[0], locations.shape[1],
                                          _pf(vectors), vectors.shape[1], 1 if overwrite else 0)
        if r:
            raise RuntimeError("no current sample")

    def batch_add_sample_from_tensor(self, tensor, offset, threshold=0.0):
        tensor = _f32(tensor)
        assert tensor.ndim == self.dim + 1
        size = np.ascontiguousarray(tensor.shape[:-1], dtype=np.int64)
        self.f["add_sample_from_tensor"](self.h, _pf(tensor), _p64(size), tensor.shape[-1],
                                         _p64(_sz(self.dim, offset)), float(threshold))

    def batch_end(self):  # the CPU implementations insert as they go: nothing left to do
        pass

    def batch_features(self):
        out = np.zeros((self.nactive(self.input_spatial), self.f["batch_planes"](self.h)), np.float32)
        if out.size:
            self.f["batch_features"](self.h, _pf(out))
        return out

    def generate_rulebooks(self, size):
        self.f["generate_rulebooks"](self.h, int(size))

    def nactive(self, spatial):
        return self.f["nactive"](self.h, _p64(_sz(self.dim, spatial)))

    def batch_size(self, spatial):
        return self.f["batch_size"](self.h, _p64(_sz(self.dim, spatial)))

    def spatial_locations(self, spatial):
        n = self.nactive(spatial)
        out = np.zeros((n, self.dim + 1), np.int64)
        if n:
            self.f["spatial_locations"](self.h, _p64(_sz(self.dim, spatial)), _p64(out))
        return out

    def _rules(self, kind, a, b=None, c=None, d=None):
        args = [_p64(_sz(self.dim, v)) if v is not None else None for v in (a, b, c, d)]
        keep = [_sz(self.dim, v) if v is not None else None for v in (a, b, c, d)]
        args = [_p64(v) for v in keep]
        k = self.f["rb_noffsets"](self.h, kind, *args)
        counts = np.zeros(k, np.int64)
        self.f["rb_counts"](self.h, kind, *args, _p64(counts))
        out = []
        for i in range(k):
            pairs = np.zeros((int(counts[i]), 2), np.int32)
            if counts[i]:
                self.f["rb_copy"](self.h, kind, *args, i, pairs.ctypes.data_as(_i32p))
            out.append(pairs)
        return out

    def submanifold_rules(self, spatial, filter_size):
        """List over filter offsets of int32 [n_k, 2] arrays of (in row, out row)."""
        return self._rules(0, spatial, filter_size)

    def strided_rules(self, in_size, out_size, filter_size, stride):
        """As above for a strided convolution; creates the out_size level."""
        return self._rules(1, in_size, out_size, filter_size, stride)

    def s2d_rules(self, spatial):
        """List over samples of int32 [n_b, 2] arrays of (row, dense offset)."""
        return self._rules(2, spatial)

    # -- forward ops ------------------------------------------------------
    def _conv(self, name, sizes, n_out_rows, x, w, bias, groups):
        x = _f32(x)
        w = _f32(w)
        bias = _f32(bias)
        n_in, n_out = w.shape[2] * w.shape[1], w.shape[3] * w.shape[1]
        out = np.zeros((n_out_rows, n_out), np.float32)
        macs = self.f[name](self.h, *[_p64(s) for s in sizes], _pf(x), _pf(out), _pf(w), _pf(bias),
                            n_in, n_out, groups)
        return out, macs

    def subm_conv(self, spatial, filter_size, x, w, bias=None):
        """w: [K, groups, nIn/groups, nOut/groups]."""
        s, f = _sz(self.dim, spatial), _sz(self.dim, filter_size)
        self.submanifold_rules(spatial, filter_size)
        return self._conv("subm_conv", (s, f), self.nactive(spatial), x, w, bias, w.shape[1])

    def conv(self, in_size, out_size, filter_size, stride, x, w, bias=None):
        self.strided_rules(in_size, out_size, filter_size, stride)
        sizes = [_sz(self.dim, v) for v in (in_size, out_size, filter_size, stride)]
        return self._conv("conv", sizes, self.nactive(out_size), x, w, bias, w.shape[1])

    def deconv(self, in_size, out_size, filter_size, stride, x, w, bias=None):
        self.strided_rules(out_size, in_size, filter_size, stride)
        sizes = [_sz(self.dim, v) for v in (in_size, out_size, filter_size, stride)]
        return self._conv("deconv", sizes, self.nactive(out_size), x, w, bias, w.shape[1])

    def maxpool(self, in_size, out_size, size, stride, x, n_features_to_drop=0):
        x = _f32(x)
        self.strided_rules(in_size, out_size, size, stride)
        sizes = [_sz(self.dim, v) for v in (in_size, out_size, size, stride)]
        planes = x.shape[1] - n_features_to_drop
        out = np.zeros((self.nactive(out_size), planes), np.float32)
        self.f["maxpool"](self.h, *[_p64(s) for s in sizes], _pf(x), x.shape[1], _pf(out), planes,
                          n_features_to_drop)
        return out

    def avgpool(self, in_size, out_size, size, stride, x, n_features_to_drop=0):
        x = _f32(x)
        self.strided_rules(in_size, out_size, size, stride)
        sizes = [_sz(self.dim, v) for v in (in_size, out_size, size, stride)]
        planes = x.shape[1] - n_features_to_drop
        out = np.zeros((self.nactive(out_size), planes), np.float32)
        self.f["avgpool"](self.h, *[_p64(s) for s in sizes], _pf(x), x.shape[1], _pf(out), planes,
                          n_features_to_drop)
        return out

    def unpool(self, in_size, out_size, size, stride, x, n_features_to_drop=0):
        """x lives on the coarse level in_size; the result on the finer level out_size."""
        x = _f32(x)
        sizes = [_sz(self.dim, v) for v in (in_size, out_size, size, stride)]
        planes = x.shape[1] - n_features_to_drop
        out = np.zeros((self.nactive(out_size), planes), np.float32)
        self.f["unpool"](self.h, *[_p64(s) for s in sizes], _pf(x), x.shape[1], _pf(out), planes,
                         n_features_to_drop)
        return out

    def nin(self, x, w, bias=None):
        """NetworkInNetwork: returns (bias + x @ w, multiply-adds)."""
        x, w, bias = _f32(x), _f32(w), _f32(bias)
        out = np.zeros((x.shape[0], w.shape[1]), np.float32)
        macs = self.f["nin"](_pf(x), _pf(out), _pf(w), _pf(bias), x.shape[0], w.shape[0], w.shape[1])
        return out, macs

    def bn_eval(self, x, mean, var, weight=None, bias=None, eps=1e-4, leakiness=1.0):
        x = _f32(x)
        out = np.zeros_like(x)
        mean, var, weight, bias = _f32(mean), _f32(var), _f32(weight), _f32(bias)
        self.f["bn_eval"](_pf(x), _pf(out), x.shape[0], x.shape[1], x.shape[1], x.shape[1],
                          _pf(mean), _pf(var), _pf(weight), _pf(bias), eps, leakiness)
        return out

    def input_fwd(self, x):
        x = _f32(x)
        hdr, _ = self.input_rules()
        out = np.zeros((int(hdr[3]), x.shape[1]), np.float32)
        self.f["input_fwd"](self.h, _pf(x), _pf(out), x.shape[1])
        return out

    def output_fwd(self, x):
        x = _f32(x)
        hdr, _ = self.input_rules()
        out = np.zeros((int(hdr[2]), x.shape[1]), np.float32)
        self.f["output_fwd"](self.h, _pf(x), _pf(out), x.shape[1])
        return out

    def s2d(self, spatial, x):
        x = _f32(x)
        s = _sz(self.dim, spatial)
        out = np.zeros((self.batch_size(spatial), x.shape[1]) + tuple(int(v) for v in s),
                       np.float32)
        self.f["s2d"](self.h, _p64(s), _pf(x), _pf(out), x.shape[1])
        return out


    # -- backward ops: each returns the gradients the reference's backward call fills ----------
    def _conv_bwd(self, name, sizes, n_in_rows, x, d_out, w, with_bias):
        x, d_out, w = _f32(x), _f32(d_out), _f32(w)
        groups = w.shape[1]
        n_in, n_out = w.shape[2] * groups, w.shape[3] * groups
        d_in = np.zeros((n_in_rows, n_in), np.float32)
        d_w = np.zeros_like(w)
        d_b = np.zeros(n_out, np.float32) if with_bias else None
        self.f[name](self.h, *[_p64(s) for s in sizes], _pf(x), _pf(d_in), _pf(d_out), _pf(w), _pf(d_w), _pf(d_b),
                     n_in, n_out, groups)
        return d_in, d_w, d_b

    def subm_conv_bwd(self, spatial, filter_size, x, d_out, w, with_bias=False):
        """(d_input, d_weight, d_bias or None) of subm_conv."""
        self.submanifold_rules(spatial, filter_size)
        sizes = (_sz(self.dim, spatial), _sz(self.dim, filter_size))
        return self._conv_bwd("subm_conv_bwd", sizes, self.nactive(spatial), x, d_out, w, with_bias)

    def conv_bwd(self, in_size, out_size, filter_size, stride, x, d_out, w, with_bias=False):
        sizes = [_sz(self.dim, v) for v in (in_size, out_size, filter_size, stride)]
        return self._conv_bwd("conv_bwd", sizes, self.nactive(in_size), x, d_out, w, with_bias)

    def deconv_bwd(self, in_size, out_size, filter_size, stride, x, d_out, w, with_bias=False):
        sizes = [_sz(self.dim, v) for v in (in_size, out_size, filter_size, stride)]
        return self._conv_bwd("deconv_bwd", sizes, self.nactive(in_size), x, d_out, w, with_bias)

    def nin_bwd(self, x, d_out, w, with_bias=False):
        x, d_out, w = _f32(x), _f32(d_out), _f32(w)
        d_in, d_w = np.zeros_like(x), np.zeros_like(w)
        d_b = np.zeros(w.shape[1], np.float32) if with_bias else None
        self.f["nin_bwd"](_pf(x), _pf(d_in), _pf(d_out), _pf(w), _pf(d_w), _pf(d_b), x.shape[0], w.shape[0], w.shape[1])
        return d_in, d_w, d_b

    def bn_train(self, x, running_mean, running_var, weight=None, bias=None, eps=1e-4, momentum=0.99,
                 leakiness=1.0):
        """Training-mode forward: (out, save_mean, save_invstd, new running_mean, new running_var)."""
        x = _f32(x)
        out = np.zeros_like(x)
        C_ = x.shape[1]
        sm, si = np.zeros(C_, np.float32), np.zeros(C_, np.float32)
        rm, rv = _f32(running_mean).copy(), _f32(running_var).copy()
        weight, bias = _f32(weight), _f32(bias)
        self.f["bn_train"](_pf(x), _pf(out), x.shape[0], C_, C_, C_, _pf(sm), _pf(si), _pf(rm), _pf(rv),
                           _pf(weight), _pf(bias), eps, momentum, leakiness)
        return out, sm, si, rm, rv

    def bn_bwd(self, x, out, d_out, save_mean, save_invstd, weight=None, leakiness=1.0, affine=True):
        """(d_input, d_weight, d_bias) of the batch norm whose forward saved mean / invstd."""
        x, out, d_out = _f32(x), _f32(out), _f32(d_out)
        C_ = x.shape[1]
        d_in = np.zeros_like(x)
        d_w = np.zeros(C_, np.float32) if affine else None
        d_b = np.zeros(C_, np.float32) if affine else None
        self.f["bn_bwd"](_pf(x), _pf(d_in), _pf(out), _pf(d_out), x.shape[0], C_, C_, C_, _pf(_f32(save_mean)),
                         _pf(_f32(save_invstd)), _pf(_f32(weight)), _pf(d_w), _pf(d_b), leakiness)
        return d_in, d_w, d_b

    def maxpool_bwd(self, in_size, out_size, size, stride, x, out, d_out, n_features_to_drop=0):
        x, out, d_out = _f32(x), _f32(out), _f32(d_out)
        sizes = [_sz(self.dim, v) for v in (in_size, out_size, size, stride)]
        d_in = np.zeros_like(x)
        self.f["maxpool_bwd"](self.h, *[_p64(s) for s in sizes], _pf(x), _pf(d_in), x.shape[1], _pf(out), _pf(d_out),
                              out.shape[1], n_features_to_drop)
        return d_in

    def avgpool_bwd(self, in_size, out_size, size, stride, in_planes, d_out, n_features_to_drop=0):
        d_out = _f32(d_out)
        sizes = [_sz(self.dim, v) for v in (in_size, out_size, size, stride)]
        d_in = np.zeros((self.nactive(in_size), in_planes), np.float32)
        self.f["avgpool_bwd"](self.h, *[_p64(s) for s in sizes], _pf(d_in), in_planes, _pf(d_out), d_out.shape[1],
                              n_features_to_drop)
        return d_in

    def unpool_bwd(self, in_size, out_size, size, stride, in_planes, d_out, n_features_to_drop=0):
        """in_size: the coarse level the unpooling's input lives on."""
        d_out = _f32(d_out)
        sizes = [_sz(self.dim, v) for v in (in_size, out_size, size, stride)]
        d_in = np.zeros((self.nactive(in_size), in_planes), np.float32)
        self.f["unpool_bwd"](self.h, *[_p64(s) for s in sizes], _pf(d_in), in_planes, _pf(d_out), d_out.shape[1],
                             n_features_to_drop)
        return d_in

    def input_bwd(self, d_out):
        d_out = _f32(d_out)
        hdr, _ = self.input_rules()
        d_in = np.zeros((int(hdr[2]), d_out.shape[1]), np.float32)
        self.f["input_bwd"](self.h, _pf(d_in), _pf(d_out), d_out.shape[1])
        return d_in

    def output_bwd(self, d_out):
        d_out = _f32(d_out)
        hdr, _ = self.input_rules()
        d_in = np.zeros((int(hdr[3]), d_out.shape[1]), np.float32)
        self.f["output_bwd"](self.h, _pf(d_in), _pf(d_out), d_out.shape[1])
        return d_in

    def bl_input_bwd(self, d_out):
        d_out = _f32(d_out)
        hdr, _ = self.bl_rules()
        d_in = np.zeros((int(hdr[2]), int(hdr[3]), d_out.shape[1]), np.float32)
        self.f["bl_input_bwd"](self.h, _pf(d_in), _pf(d_out), d_out.shape[1])
        return d_in

    def bl_output_bwd(self, d_out):
        d_out = _f32(d_out)
        hdr, _ = self.bl_rules()
        flat = np.ascontiguousarray(d_out.reshape(-1, d_out.shape[-1]))
        d_in = np.zeros((int(hdr[4]), d_out.shape[-1]), np.float32)
        self.f["bl_output_bwd"](self.h, _pf(d_in), _pf(flat), d_out.shape[-1])
        return d_in

    def active_pooling(self, spatial, x, average=False):
        """[batch, planes], or None from the compiled reference where its rule builder
        (Metadata/ActivePoolingRules.h:29) would not return: a sample with other than one site."""
        x = _f32(x)
        out = np.zeros((self.batch_size(spatial), x.shape[1]), np.float32)
        ok = self.f["active_pooling"](self.h, _p64(_sz(self.dim, spatial)), _pf(x), _pf(out), x.shape[1], int(average))
        return out if ok else None

    def active_pooling_bwd(self, spatial, d_out, average=False):
        d_out = _f32(d_out)
        d_in = np.zeros((self.nactive(spatial), d_out.shape[1]), np.float32)
        ok = self.f["active_pooling_bwd"](self.h, _p64(_sz(self.dim, spatial)), _pf(d_in), _pf(d_out), d_out.shape[1],
                                          int(average))
        return d_in if ok else None

    def s2d_bwd(self, spatial, d_out):
        d_out = _f32(d_out)
        s = _sz(self.dim, spatial)
        d_in = np.zeros((self.nactive(spatial), d_out.shape[1]), np.float32)
        self.f["s2d_bwd"](self.h, _p64(s), _pf(d_in), _pf(d_out), d_out.shape[1])
        return d_in


def canon_rules(rules, loc_in, loc_out):
    """Canonical form of a rulebook: a sorted int64 array of rows
    (offset, in-site coords+batch, out-site coords+batch), independent of how
    either side numbers its rows."""
    rows = []
    for k, pairs in enumerate(rules):
        if len(pairs) == 0:
            continue
        a = loc_in[pairs[:, 0]]
        b = loc_out[pairs[:, 1]]
        rows.append(np.concatenate([np.full((len(pairs), 1), k, np.int64), a, b], axis=1))
    if not rows:
        return np.zeros((0, 1 + loc_in.shape[1] + loc_out.shape[1]), np.int64)
    allr = np.concatenate(rows, axis=0)
    order = np.lexsort(allr.T[::-1])
    return allr[order]


def canon_rows(loc):
    """Permutation that sorts sites by (batch, coords): use it to compare feature
    matrices of two implementations that number rows differently."""
    key = np.concatenate([loc[:, -1:], loc[:, :-1]], axis=1)
    return np.lexsort(key.T[::-1])
