"""The C ABI of libscn_hip.so behind the interface of oracle.cpu_path.CpuPath, so that the
checks written for the CPU implementations run unchanged on the GPU library.  numpy in,
numpy out; device memory and the stream come from torch."""
import ctypes as C

import numpy as np
import torch

from sparseconvnet_amd import _lib


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(a, dtype):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=dtype).cuda().contiguous()


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None and t.numel() else C.c_void_p(0)


class HipPath:
    def __init__(self, dim):
        self.L = _lib.lib()
        self.dim = dim
        self.h = self.L.scn_md_create(dim)
        if not self.h:
            raise _lib.ScnError(self.L.scn_last_error().decode())

    def set_bf16(self, enable=True):
        _lib.check(self.L.scn_md_set_bf16(self.h, 1 if enable else 0))

    def __del__(self):
        if getattr(self, "h", None):
            self.L.scn_md_destroy(self.h)
            self.h = None

    def _s(self, x):
        return _lib.sizes(self.dim, x) if x is not None else None

    # -- metadata ---------------------------------------------------------
    host_coords = False  # True: coordinates are handed over in host memory (scn_md_input_layer_host)

    def input_layer(self, spatial, coords, batch_size=0, mode=3):
        coords = np.ascontiguousarray(coords, dtype=np.int64)
        n = C.c_int64(0)
        if self.host_coords:
            _lib.check(self.L.scn_md_input_layer_host(self.h, self._s(spatial), C.c_void_p(coords.ctypes.data),
                                                      coords.shape[0], coords.shape[1], batch_size, mode, _stream(),
                                                      C.byref(n)))
            return n.value
        c = _dev(coords, torch.int64)
        _lib.check(self.L.scn_md_input_layer(self.h, self._s(spatial), _ptr(c), coords.shape[0],
                                             coords.shape[1], batch_size, mode, _stream(), C.byref(n)))
        return n.value

    def input_rules(self):
        hdr = (C.c_int32 * 4)()
        _lib.check(self.L.scn_md_input_rules_header(self.h, hdr))
        mode, max_active, n_in, n_out = [int(v) for v in hdr]
        rows = torch.zeros((n_out, 1 + max_active), dtype=torch.int32, device="cuda")
        if mode != 0 and n_out:
            _lib.check(self.L.scn_md_input_rules(self.h, _ptr(rows), _stream()))
        return np.array(list(hdr), np.int32), rows.cpu().numpy()

    def bl_input_layer(self, spatial, coords, mode=3):
        coords = np.ascontiguousarray(coords, dtype=np.int64)
        c = _dev(coords, torch.int64)
        n = C.c_int64(0)
        _lib.check(self.L.scn_md_bl_input_layer(self.h, self._s(spatial), _ptr(c), coords.shape[0],
                                                coords.shape[1], mode, _stream(), C.byref(n)))
        return n.value

    def bl_rules(self):
        hdr = (C.c_int32 * 5)()
        _lib.check(self.L.scn_md_bl_rules_header(self.h, hdr))
        mode, max_active, _, _, n_out = [int(v) for v in hdr]
        rows = torch.zeros((n_out, 1 + max_active), dtype=torch.int32, device="cuda")
        if mode != 0 and n_out:
            _lib.check(self.L.scn_md_input_rules(self.h, _ptr(rows), _stream()))
        return np.array(list(hdr), np.int32), rows.cpu().numpy()

    def bl_input_fwd(self, x):
        hdr, _ = self.bl_rules()
        xd = _dev(np.ascontiguousarray(x.reshape(-1, x.shape[-1])), torch.float32)
        out = torch.full((int(hdr[4]), x.shape[-1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_input_layer_fwd(self.h, _ptr(xd), _ptr(out), x.shape[-1], _stream()))
        return out.cpu().numpy()

    def bl_output_fwd(self, x):
        hdr, _ = self.bl_rules()
        xd = _dev(x, torch.float32)
        out = torch.full((int(hdr[2]), int(hdr[3]), x.shape[1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_output_layer_fwd(self.h, _ptr(xd), _ptr(out), x.shape[1], _stream()))
        return out.cpu().numpy()

    # point-at-a-time input: the calls collect, batch_end hands everything to the library
    def batch_begin(self, spatial):
        self.input_spatial = np.broadcast_to(np.asarray(spatial, np.int64), (self.dim,)).copy()
        self._b_coords, self._b_vectors, self._b_flags = [], [], []
        self._b_samples, self._b_current, self._b_feats = 0, -1, None

    def batch_add_sample(self):
        self._b_samples += 1
        self._b_current = self._b_samples - 1

    def batch_set_locations(self, locations, vectors, overwrite=False):
        locations = np.ascontiguousarray(locations, dtype=np.int64)
        vectors = np.ascontiguousarray(vectors, dtype=np.float32)
        if locations.shape[1] == self.dim:
            if self._b_current < 0:
                raise RuntimeError("no current sample")
            locations = np.concatenate([locations, np.full((len(locations), 1), self._b_current, np.int64)], 1)
        elif len(locations):
            self._b_samples = max(self._b_samples, int(locations[:, -1].max()) + 1)
        self._b_coords.append(locations)
        self._b_vectors.append(vectors)
        self._b_flags.append(np.full(len(locations), 1 if overwrite else 0, np.uint8))

    def batch_add_sample_from_tensor(self, tensor, offset, threshold=0.0):
        tensor = np.ascontiguousarray(tensor, dtype=np.float32)
        offset = np.broadcast_to(np.asarray(offset, np.int64), (self.dim,))
        self._b_samples += 1
        cells = np.argwhere((np.abs(tensor) > threshold).any(-1))
        where = cells + offset
        inside = ((where >= 0) & (where < self.input_spatial)).all(1)
        cells, where = cells[inside], where[inside]
        self._b_coords.append(np.concatenate([where, np.full((len(where), 1), self._b_samples - 1, np.int64)], 1))
        self._b_vectors.append(tensor[tuple(cells.T)].reshape(len(cells), tensor.shape[-1]))
        self._b_flags.append(np.zeros(len(where), np.uint8))

    def batch_end(self):
        coords = np.concatenate(self._b_coords) if self._b_coords else np.zeros((0, self.dim + 1), np.int64)
        planes = self._b_vectors[0].shape[1] if self._b_vectors else 0
        vectors = np.concatenate(self._b_vectors) if self._b_vectors else np.zeros((0, planes), np.float32)
        flags = np.concatenate(self._b_flags) if self._b_flags else np.zeros(0, np.uint8)
        c, v = _dev(coords, torch.int64), _dev(vectors, torch.float32)
        f = _dev(flags, torch.uint8) if flags.any() else None
        n = C.c_int64(0)
        _lib.check(self.L.scn_md_input_batch(self.h, self._s(self.input_spatial), _ptr(c), _ptr(f), len(coords),
                                             self.dim + 1, self._b_samples, _stream(), C.byref(n)))
        out = torch.full((n.value, planes), float("nan"), dtype=torch.float32, device="cuda")
        if planes:
            _lib.check(self.L.scn_input_layer_fwd(self.h, _ptr(v), _ptr(out), planes, _stream()))
        self._b_feats = out.cpu().numpy()

    def batch_features(self):
        return self._b_feats

    def generate_rulebooks(self, size):
        _lib.check(self.L.scn_md_generate_rulebooks(self.h, int(size), _stream()))

    def nactive(self, spatial):
        n = C.c_int64(0)
        _lib.check(self.L.scn_md_nactive(self.h, self._s(spatial), C.byref(n)))
        return n.value

    def batch_size(self, spatial):
        b = C.c_int(0)
        _lib.check(self.L.scn_md_batch_size(self.h, self._s(spatial), C.byref(b)))
        return b.value

    def spatial_locations(self, spatial):
        n = self.nactive(spatial)
        out = torch.zeros((n, self.dim + 1), dtype=torch.int64, device="cuda")
        if n:
            _lib.check(self.L.scn_md_spatial_locations(self.h, self._s(spatial), _ptr(out), _stream()))
        return out.cpu().numpy()

    def _rules(self, kind, a, b=None, c=None, d=None):
        args = [self._s(v) for v in (a, b, c, d)]
        cnt = C.c_int(0)
        _lib.check(self.L.scn_rules_count(self.h, kind, *args, _stream(), C.byref(cnt)))
        sizes = (C.c_int64 * max(1, cnt.value))()
        _lib.check(self.L.scn_rules_sizes(self.h, kind, *args, _stream(), sizes))
        out = []
        for k in range(cnt.value):
            pairs = torch.zeros((int(sizes[k]), 2), dtype=torch.int32, device="cuda")
            if sizes[k]:
                _lib.check(self.L.scn_rules_export(self.h, kind, *args, k, _ptr(pairs), _stream()))
            out.append(pairs.cpu().numpy())
        return out

    def submanifold_rules(self, spatial, filter_size):
        return self._rules(0, spatial, filter_size)

    def strided_rules(self, in_size, out_size, filter_size, stride):
        return self._rules(1, in_size, out_size, filter_size, stride)

    def s2d_rules(self, spatial):
        return self._rules(2, spatial)

    # -- forward ops ------------------------------------------------------
    def _conv(self, kind, sizes, n_rows, x, w, bias, bn=None, post=None):
        """bn / post: None or dict(mean, var, weight, bias, eps, leakiness) of a batch norm in
        front of / behind the convolution: the fused entry point scn_conv_bn_fwd."""
        groups = w.shape[1]
        n_in, n_out = w.shape[2] * groups, w.shape[3] * groups
        xd, wd = _dev(x, torch.float32), _dev(w, torch.float32)
        bd = _dev(bias, torch.float32) if bias is not None else None
        out = torch.full((n_rows, n_out), float("nan"), dtype=torch.float32, device="cuda")
        macs = C.c_double(0)
        tail = (_ptr(xd), _ptr(out), _ptr(wd), _ptr(bd), n_in, n_out, groups)
        if bn is None and post is None:
            fn = (self.L.scn_subm_conv_fwd, self.L.scn_conv_fwd, self.L.scn_deconv_fwd)[kind]
            _lib.check(fn(self.h, *sizes, *tail, _stream(), C.byref(macs)))
        else:
            keep = []

            def params(p):
                if p is None:
                    return None
                t = [_dev(p[k], torch.float32) if p.get(k) is not None else None
                     for k in ("mean", "var", "weight", "bias")]
                keep.extend(t)
                return C.byref(_lib.BnParams(*[_ptr(v) for v in t], p["eps"], p["leakiness"]))
            sz = list(sizes) + [None] * (4 - len(sizes))
            _lib.check(self.L.scn_conv_bn_fwd(self.h, kind, *sz, *tail, params(bn), params(post), _stream(),
                                              C.byref(macs)))
        return out.cpu().numpy(), macs.value

    def subm_conv(self, spatial, filter_size, x, w, bias=None, bn=None, post=None):
        _lib.check(self.L.scn_md_submanifold_rules(self.h, self._s(spatial), self._s(filter_size),
                                                   _stream()))
        return self._conv(0, (self._s(spatial), self._s(filter_size)), self.nactive(spatial), x, w, bias, bn, post)

    def conv(self, in_size, out_size, filter_size, stride, x, w, bias=None, bn=None, post=None):
        sizes = [self._s(v) for v in (in_size, out_size, filter_size, stride)]
        _lib.check(self.L.scn_md_strided_rules(self.h, *sizes, _stream()))
        return self._conv(1, sizes, self.nactive(out_size), x, w, bias, bn, post)

    def deconv(self, in_size, out_size, filter_size, stride, x, w, bias=None, bn=None, post=None):
        sizes = [self._s(v) for v in (in_size, out_size, filter_size, stride)]
        rb = [self._s(v) for v in (out_size, in_size, filter_size, stride)]
        _lib.check(self.L.scn_md_strided_rules(self.h, *rb, _stream()))
        return self._conv(2, sizes, self.nactive(out_size), x, w, bias, bn, post)

    def nin(self, x, w, bias=None):
        xd, wd = _dev(x, torch.float32), _dev(w, torch.float32)
        bd = _dev(bias, torch.float32) if bias is not None else None
        out = torch.full((x.shape[0], w.shape[1]), float("nan"), dtype=torch.float32, device="cuda")
        macs = C.c_double(0)
        _lib.check(self.L.scn_nin_fwd(self.h, _ptr(xd), _ptr(out), _ptr(wd), _ptr(bd), x.shape[0], w.shape[0],
                                      w.shape[1], _stream(), C.byref(macs)))
        return out.cpu().numpy(), macs.value

    def maxpool(self, in_size, out_size, size, stride, x, n_features_to_drop=0):
        sizes = [self._s(v) for v in (in_size, out_size, size, stride)]
        _lib.check(self.L.scn_md_strided_rules(self.h, *sizes, _stream()))
        xd = _dev(x, torch.float32)
        planes = x.shape[1] - n_features_to_drop
        out = torch.full((self.nactive(out_size), planes), float("nan"), dtype=torch.float32,
                         device="cuda")
        _lib.check(self.L.scn_maxpool_fwd(self.h, *sizes, _ptr(xd), x.shape[1], _ptr(out), planes,
                                          n_features_to_drop, _stream()))
        return out.cpu().numpy()

    def avgpool(self, in_size, out_size, size, stride, x, n_features_to_drop=0):
        sizes = [self._s(v) for v in (in_size, out_size, size, stride)]
        _lib.check(self.L.scn_md_strided_rules(self.h, *sizes, _stream()))
        xd = _dev(x, torch.float32)
        planes = x.shape[1] - n_features_to_drop
        out = torch.full((self.nactive(out_size), planes), float("nan"), dtype=torch.float32,
                         device="cuda")
        _lib.check(self.L.scn_avgpool_fwd(self.h, *sizes, _ptr(xd), x.shape[1], _ptr(out), planes,
                                          n_features_to_drop, _stream()))
        return out.cpu().numpy()

    def unpool(self, in_size, out_size, size, stride, x, n_features_to_drop=0):
        sizes = [self._s(v) for v in (in_size, out_size, size, stride)]
        xd = _dev(x, torch.float32)
        planes = x.shape[1] - n_features_to_drop
        out = torch.full((self.nactive(out_size), planes), float("nan"), dtype=torch.float32,
                         device="cuda")
        _lib.check(self.L.scn_unpool_fwd(self.h, *sizes, _ptr(xd), x.shape[1], _ptr(out), planes,
                                         n_features_to_drop, _stream()))
        return out.cpu().numpy()

    def bn_eval(self, x, mean, var, weight=None, bias=None, eps=1e-4, leakiness=1.0):
        xd = _dev(x, torch.float32)
        out = torch.full_like(xd, float("nan"))
        md, vd = _dev(mean, torch.float32), _dev(var, torch.float32)
        gd = _dev(weight, torch.float32) if weight is not None else None
        bd = _dev(bias, torch.float32) if bias is not None else None
        _lib.check(self.L.scn_bn_eval_fwd(_ptr(xd), _ptr(out), x.shape[0], x.shape[1], x.shape[1],
                                          x.shape[1], _ptr(md), _ptr(vd), _ptr(gd), _ptr(bd), eps,
                                          leakiness, _stream()))
        return out.cpu().numpy()

    def input_fwd(self, x):
        hdr = self._hdr()
        xd = _dev(x, torch.float32)
        out = torch.full((int(hdr[3]), x.shape[1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_input_layer_fwd(self.h, _ptr(xd), _ptr(out), x.shape[1], _stream()))
        return out.cpu().numpy()

    def _hdr(self):
        hdr = (C.c_int32 * 4)()
        _lib.check(self.L.scn_md_input_rules_header(self.h, hdr))
        return [int(v) for v in hdr]

    def output_fwd(self, x):
        hdr = self._hdr()
        xd = _dev(x, torch.float32)
        out = torch.full((hdr[2], x.shape[1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_output_layer_fwd(self.h, _ptr(xd), _ptr(out), x.shape[1], _stream()))
        return out.cpu().numpy()

    def s2d(self, spatial, x):
        s = [int(v) for v in self._s(spatial)]
        xd = _dev(x, torch.float32)
        out = torch.full([self.batch_size(spatial), x.shape[1]] + s, float("nan"), dtype=torch.float32,
                         device="cuda")
        _lib.check(self.L.scn_s2d_fwd(self.h, self._s(spatial), _ptr(xd), _ptr(out), x.shape[1],
                                      _stream()))
        return out.cpu().numpy()

    # -- backward ops (same interface as oracle.cpu_path.CpuPath) ------------------------------
    def _conv_bwd(self, fn, sizes, n_in_rows, x, d_out, w, with_bias):
        groups = w.shape[1]
        n_in, n_out = w.shape[2] * groups, w.shape[3] * groups
        xd, dd, wd = _dev(x, torch.float32), _dev(d_out, torch.float32), _dev(w, torch.float32)
        d_in = torch.full((n_in_rows, n_in), float("nan"), dtype=torch.float32, device="cuda")
        d_w = torch.full_like(wd, float("nan"))
        d_b = torch.full((n_out,), float("nan"), dtype=torch.float32, device="cuda") if with_bias else None
        _lib.check(fn(self.h, *sizes, _ptr(xd), _ptr(d_in), _ptr(dd), _ptr(wd), _ptr(d_w), _ptr(d_b), n_in, n_out,
                      groups, _stream()))
        return d_in.cpu().numpy(), d_w.cpu().numpy(), (d_b.cpu().numpy() if with_bias else None)

    def subm_conv_bwd(self, spatial, filter_size, x, d_out, w, with_bias=False):
        sizes = (self._s(spatial), self._s(filter_size))
        return self._conv_bwd(self.L.scn_subm_conv_bwd, sizes, self.nactive(spatial), x, d_out, w, with_bias)

    def conv_bwd(self, in_size, out_size, filter_size, stride, x, d_out, w, with_bias=False):
        sizes = [self._s(v) for v in (in_size, out_size, filter_size, stride)]
        return self._conv_bwd(self.L.scn_conv_bwd, sizes, self.nactive(in_size), x, d_out, w, with_bias)

    def deconv_bwd(self, in_size, out_size, filter_size, stride, x, d_out, w, with_bias=False):
        sizes = [self._s(v) for v in (in_size, out_size, filter_size, stride)]
        return self._conv_bwd(self.L.scn_deconv_bwd, sizes, self.nactive(in_size), x, d_out, w, with_bias)

    def nin_bwd(self, x, d_out, w, with_bias=False):
        xd, dd, wd = _dev(x, torch.float32), _dev(d_out, torch.float32), _dev(w, torch.float32)
        d_in, d_w = torch.full_like(xd, float("nan")), torch.full_like(wd, float("nan"))
        d_b = torch.full((w.shape[1],), float("nan"), dtype=torch.float32, device="cuda") if with_bias else None
        _lib.check(self.L.scn_nin_bwd(self.h, _ptr(xd), _ptr(d_in), _ptr(dd), _ptr(wd), _ptr(d_w), _ptr(d_b), x.shape[0],
                                      w.shape[0], w.shape[1], _stream()))
        return d_in.cpu().numpy(), d_w.cpu().numpy(), (d_b.cpu().numpy() if with_bias else None)

    def bn_train(self, x, running_mean, running_var, weight=None, bias=None, eps=1e-4, momentum=0.99, leakiness=1.0):
        xd = _dev(x, torch.float32)
        out = torch.full_like(xd, float("nan"))
        C_ = x.shape[1]
        sm, si = torch.zeros(C_, device="cuda"), torch.zeros(C_, device="cuda")
        rm, rv = _dev(running_mean, torch.float32).clone(), _dev(running_var, torch.float32).clone()
        gd = _dev(weight, torch.float32) if weight is not None else None
        bd = _dev(bias, torch.float32) if bias is not None else None
        _lib.check(self.L.scn_bn_train_fwd(self.h, _ptr(xd), _ptr(out), x.shape[0], C_, C_, C_, _ptr(sm), _ptr(si), _ptr(rm),
                                           _ptr(rv), _ptr(gd), _ptr(bd), eps, momentum, leakiness, _stream()))
        return tuple(t.cpu().numpy() for t in (out, sm, si, rm, rv))

    def bn_bwd(self, x, out, d_out, save_mean, save_invstd, weight=None, leakiness=1.0, affine=True):
        xd, od, dd = _dev(x, torch.float32), _dev(out, torch.float32), _dev(d_out, torch.float32)
        C_ = x.shape[1]
        d_in = torch.full_like(xd, float("nan"))
        d_w = torch.full((C_,), float("nan"), device="cuda") if affine else None
        d_b = torch.full((C_,), float("nan"), device="cuda") if affine else None
        gd = _dev(weight, torch.float32) if weight is not None else None
        sm, si = _dev(save_mean, torch.float32), _dev(save_invstd, torch.float32)
        _lib.check(self.L.scn_bn_bwd(self.h, _ptr(xd), _ptr(d_in), _ptr(od), _ptr(dd), x.shape[0], C_, C_, C_, _ptr(sm),
                                     _ptr(si), _ptr(gd), _ptr(d_w), _ptr(d_b), leakiness, _stream()))
        return d_in.cpu().numpy(), (d_w.cpu().numpy() if affine else None), (d_b.cpu().numpy() if affine else None)

    def maxpool_bwd(self, in_size, out_size, size, stride, x, out, d_out, n_features_to_drop=0):
        sizes = [self._s(v) for v in (in_size, out_size, size, stride)]
        xd, od, dd = _dev(x, torch.float32), _dev(out, torch.float32), _dev(d_out, torch.float32)
        d_in = torch.full_like(xd, float("nan"))
        _lib.check(self.L.scn_maxpool_bwd(self.h, *sizes, _ptr(xd), _ptr(d_in), x.shape[1], _ptr(od), _ptr(dd),
                                          out.shape[1], n_features_to_drop, _stream()))
        return d_in.cpu().numpy()

    def _pool_bwd(self, fn, in_size, out_size, size, stride, in_planes, d_out, n_features_to_drop):
        sizes = [self._s(v) for v in (in_size, out_size, size, stride)]
        dd = _dev(d_out, torch.float32)
        d_in = torch.full((self.nactive(in_size), in_planes), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(fn(self.h, *sizes, _ptr(d_in), in_planes, _ptr(dd), d_out.shape[1], n_features_to_drop, _stream()))
        return d_in.cpu().numpy()

    def avgpool_bwd(self, in_size, out_size, size, stride, in_planes, d_out, n_features_to_drop=0):
        return self._pool_bwd(self.L.scn_avgpool_bwd, in_size, out_size, size, stride, in_planes, d_out,
                              n_features_to_drop)

    def unpool_bwd(self, in_size, out_size, size, stride, in_planes, d_out, n_features_to_drop=0):
        return self._pool_bwd(self.L.scn_unpool_bwd, in_size, out_size, size, stride, in_planes, d_out,
                              n_features_to_drop)

    def input_bwd(self, d_out):
        hdr = self._hdr()
        dd = _dev(d_out, torch.float32)
        d_in = torch.full((hdr[2], d_out.shape[1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_input_layer_bwd(self.h, _ptr(d_in), _ptr(dd), d_out.shape[1], _stream()))
        return d_in.cpu().numpy()

    def output_bwd(self, d_out):
        hdr = self._hdr()
        dd = _dev(d_out, torch.float32)
        d_in = torch.full((hdr[3], d_out.shape[1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_output_layer_bwd(self.h, _ptr(d_in), _ptr(dd), d_out.shape[1], _stream()))
        return d_in.cpu().numpy()

    def bl_input_bwd(self, d_out):
        hdr, _ = self.bl_rules()
        dd = _dev(d_out, torch.float32)
        d_in = torch.full((int(hdr[2]), int(hdr[3]), d_out.shape[1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_input_layer_bwd(self.h, _ptr(d_in), _ptr(dd), d_out.shape[1], _stream()))
        return d_in.cpu().numpy()

    def bl_output_bwd(self, d_out):
        hdr, _ = self.bl_rules()
        dd = _dev(np.ascontiguousarray(d_out.reshape(-1, d_out.shape[-1])), torch.float32)
        d_in = torch.full((int(hdr[4]), d_out.shape[-1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_output_layer_bwd(self.h, _ptr(d_in), _ptr(dd), d_out.shape[-1], _stream()))
        return d_in.cpu().numpy()

    def active_pooling(self, spatial, x, average=False):
        xd = _dev(x, torch.float32)
        out = torch.full((self.batch_size(spatial), x.shape[1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_active_pooling_fwd(self.h, self._s(spatial), _ptr(xd), _ptr(out), x.shape[1], int(average),
                                                 _stream()))
        return out.cpu().numpy()

    def active_pooling_bwd(self, spatial, d_out, average=False):
        dd = _dev(d_out, torch.float32)
        d_in = torch.full((self.nactive(spatial), d_out.shape[1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_active_pooling_bwd(self.h, self._s(spatial), _ptr(d_in), _ptr(dd), d_out.shape[1],
                                                 int(average), _stream()))
        return d_in.cpu().numpy()

    def s2d_bwd(self, spatial, d_out):
        dd = _dev(d_out, torch.float32)
        d_in = torch.full((self.nactive(spatial), d_out.shape[1]), float("nan"), dtype=torch.float32, device="cuda")
        _lib.check(self.L.scn_s2d_bwd(self.h, self._s(spatial), _ptr(d_in), _ptr(dd), d_out.shape[1], _stream()))
        return d_in.cpu().numpy()
