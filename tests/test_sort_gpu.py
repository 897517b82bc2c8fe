"""The rulebook builders' radix sort through the C ABI against numpy's stable argsort: sizes around
the one-workgroup limit and the tile size, ragged tails, 1 to 64 key bits, repeated keys (stability
is what makes the input layer's first-occurrence row numbers come out)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,bits", [(1, 8), (63, 3), (4096, 16), (4097, 16), (2048 * 3 + 5, 24), (100003, 36),
                                    (1 << 20, 40), (300000, 64), (70000, 1), (5000, 9), (2500000, 33),
                                    (1000, 27), (4095, 35), (3001, 64), (2, 1)])
def test_sort_pairs(n, bits):
    import torch
    from sparseconvnet_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(n + bits)
    span = min(bits, 12) if n % 2 else bits  # odd sizes: few distinct keys, many repeats
    keys = rng.integers(0, 1 << min(span, 63), size=n, dtype=np.uint64)
    if bits == 64:
        keys |= rng.integers(0, 2, size=n, dtype=np.uint64) << np.uint64(63)
    junk = rng.integers(0, 1 << 20, size=n, dtype=np.uint64) << np.uint64(bits) if bits < 44 else np.zeros(n, np.uint64)
    keys_all = keys | junk  # bits above end_bit must not matter
    vals = np.arange(n, dtype=np.int32)
    kin = torch.as_tensor(keys_all.view(np.int64)).cuda()
    vin = torch.as_tensor(vals).cuda()
    kout, vout = torch.empty_like(kin), torch.empty_like(vin)
    h = L.scn_md_create(3)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(L.scn_sort_pairs(h, C.c_void_p(kin.data_ptr()), C.c_void_p(kout.data_ptr()), C.c_void_p(vin.data_ptr()),
                                C.c_void_p(vout.data_ptr()), n, bits, stream))
    torch.cuda.synchronize()
    mask = np.uint64((1 << bits) - 1) if bits < 64 else np.uint64(0xFFFFFFFFFFFFFFFF)
    order = np.argsort(keys_all & mask, kind="stable")
    assert (vout.cpu().numpy() == vals[order]).all()
    assert (kout.cpu().numpy().view(np.uint64) == keys_all[order]).all()
    assert (kin.cpu().numpy().view(np.uint64) == keys_all).all(), "the input arrays must not be written"
    L.scn_md_destroy(h)
