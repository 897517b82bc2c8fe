"""The allocation-free entry point scn_subm_conv_fwd_noalloc, called through the C ABI, against
scn_subm_conv_fwd on the same inputs (fp32: 1e-4 relative, 1e-5 absolute): two calls in a row
on the static scratch, the second with a smaller input, every kernel family, and no device
allocation by the library in between."""
import ctypes as C

import numpy as np
import pytest

import checks
from sparseconvnet_amd import synthetic

pytestmark = pytest.mark.gpu


def _ptr(t):
    return C.c_void_p(t.data_ptr())


def test_noalloc_matches_the_allocating_entry_point():
    import torch
    from sparseconvnet_amd import _lib
    L = _lib.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator(device="cuda").manual_seed(70)
    scenes = []
    # a large scene, then a smaller one (fewer sites: the small level's taps are split over workgroups)
    for seed, target, spatial in ((7100, 60000, 512), (7101, 3000, 128)):
        coords = synthetic.room_scene(seed=seed, target=target, spatial=spatial)
        cd = torch.as_tensor(coords).cuda()
        h = L.scn_md_create(3)
        n = C.c_int64(0)
        sp, fs = _lib.sizes(3, spatial), _lib.sizes(3, 3)
        _lib.check(L.scn_md_input_layer(h, sp, _ptr(cd), len(coords), 4, 0, 0, stream, C.byref(n)))
        scenes.append((h, sp, fs, int(n.value), cd))
    try:
        h0, sp0, fs0, n0, _ = scenes[0]
        x = torch.randn((n0, 8), device="cuda", generator=g)
        w = torch.randn((27, 1, 8, 8), device="cuda", generator=g)
        y = torch.empty((n0, 8), device="cuda")
        assert L.scn_subm_conv_fwd_noalloc(h0, sp0, fs0, _ptr(x), _ptr(y), _ptr(w), None, 8, 8, stream) != 0
        assert b"rulebook first" in L.scn_last_error()
        for h, sp, fs, n, _ in scenes:
            _lib.check(L.scn_md_submanifold_rules(h, sp, fs, stream))
        # every kernel family: four-channel resident, resident, row-owner, LDS-tiled, generic widths
        pairs = [(3, 32), (32, 32), (16, 16), (64, 64), (96, 128), (256, 256), (128, 160), (30, 50)]
        cases = []
        for cin, cout in pairs:
            for h, sp, fs, n, _ in scenes:  # the larger input first, then the smaller one
                x = torch.randn((n, cin), device="cuda", generator=g)
                w = torch.randn((27, 1, cin, cout), device="cuda", generator=g) * (2.0 / (cin * 27)) ** 0.5
                b = torch.randn((cout,), device="cuda", generator=g)
                want = torch.full((n, cout), float("nan"), device="cuda")
                macs = C.c_double(0)
                _lib.check(L.scn_subm_conv_fwd(h, sp, fs, _ptr(x), _ptr(want), _ptr(w), _ptr(b), cin, cout, 1, stream,
                                               C.byref(macs)))
                got = torch.full((n, cout), float("nan"), device="cuda")
                cases.append((h, sp, fs, x, w, b, want, got, cin, cout, macs.value))
        torch.cuda.synchronize()
        taken = C.c_double(0)
        for h, *_ in scenes:
            _lib.check(L.scn_md_take_macs(h, stream, C.byref(taken)))
        before = C.c_int64(0)
        _lib.check(L.scn_cache_stats(None, None, None, C.byref(before)))
        for h, sp, fs, x, w, b, want, got, cin, cout, _ in cases:  # back to back on the one scratch array
            _lib.check(L.scn_subm_conv_fwd_noalloc(h, sp, fs, _ptr(x), _ptr(got), _ptr(w), _ptr(b), cin, cout, stream))
        after = C.c_int64(0)
        _lib.check(L.scn_cache_stats(None, None, None, C.byref(after)))
        assert after.value == before.value, "the allocation-free entry point allocated device memory"
        torch.cuda.synchronize()
        for h, sp, fs, x, w, b, want, got, cin, cout, _ in cases:
            checks.assert_close(got.cpu().numpy(), want.cpu().numpy(), "%d -> %d on %d rows" % (cin, cout, x.shape[0]))
        # the multiply-adds were added to the handles' running totals
        total = 0.0
        for h, *_ in scenes:
            _lib.check(L.scn_md_take_macs(h, stream, C.byref(taken)))
            total += taken.value
        assert total == sum(c[-1] for c in cases)
        # weights beyond the scratch's 8 MiB are refused with a message, nothing runs
        h, sp, fs, n, _ = scenes[1]
        x = torch.randn((n, 512), device="cuda", generator=g)
        w = torch.randn((27, 1, 512, 256), device="cuda", generator=g)
        y = torch.empty((n, 256), device="cuda")
        assert L.scn_subm_conv_fwd_noalloc(h, sp, fs, _ptr(x), _ptr(y), _ptr(w), None, 512, 256, stream) != 0
        assert b"8 MiB" in L.scn_last_error()
        # more than 256 output planes would need an allocated copy of the weights: refused as well
        x = torch.randn((n, 64), device="cuda", generator=g)
        w = torch.randn((27, 1, 64, 320), device="cuda", generator=g)
        y = torch.empty((n, 320), device="cuda")
        assert L.scn_subm_conv_fwd_noalloc(h, sp, fs, _ptr(x), _ptr(y), _ptr(w), None, 64, 320, stream) != 0
        assert b"256 output planes" in L.scn_last_error()
        # A handle that has only had its rulebook built (no allocating convolution has warmed any of
        # its buffers): the allocation counter must not move over calls of every kernel family.
        coords = synthetic.room_scene(seed=7102, target=20000, spatial=256)
        cd = torch.as_tensor(coords).cuda()
        hf = L.scn_md_create(3)
        scenes.append((hf, None, None, 0, cd))
        nf = C.c_int64(0)
        spf = _lib.sizes(3, 256)
        _lib.check(L.scn_md_input_layer(hf, spf, _ptr(cd), len(coords), 4, 0, 0, stream, C.byref(nf)))
        _lib.check(L.scn_md_submanifold_rules(hf, spf, fs, stream))
        fresh = []
        for cin, cout in pairs:
            x = torch.randn((nf.value, cin), device="cuda", generator=g)
            w = torch.randn((27, 1, cin, cout), device="cuda", generator=g) * (2.0 / (cin * 27)) ** 0.5
            fresh.append((x, w, torch.empty((nf.value, cout), device="cuda"), torch.empty((nf.value, cout), device="cuda"), cin, cout))
        torch.cuda.synchronize()
        _lib.check(L.scn_cache_stats(None, None, None, C.byref(before)))
        for x, w, got, _, cin, cout in fresh:
            _lib.check(L.scn_subm_conv_fwd_noalloc(hf, spf, fs, _ptr(x), _ptr(got), _ptr(w), None, cin, cout, stream))
        _lib.check(L.scn_cache_stats(None, None, None, C.byref(after)))
        assert after.value == before.value, "the allocation-free entry point allocated device memory on a fresh handle"
        for x, w, got, want, cin, cout in fresh:
            _lib.check(L.scn_subm_conv_fwd(hf, spf, fs, _ptr(x), _ptr(want), _ptr(w), None, cin, cout, 1, stream, None))
        torch.cuda.synchronize()
        for x, w, got, want, cin, cout in fresh:
            checks.assert_close(got.cpu().numpy(), want.cpu().numpy(), "fresh handle %d -> %d" % (cin, cout))
    finally:
        for h, *_ in scenes:
            L.scn_md_destroy(h)
