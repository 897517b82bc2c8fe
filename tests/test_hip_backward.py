"""Backward pass of the HIP library through its C ABI: the independent checks of tests/checks.py
(torch.autograd through the dense equivalents) and the CPU oracle on the same seeded inputs over
every kernel family's channel range.  Gradients within 1e-4 relative / 1e-5 absolute (fp32)."""
import numpy as np
import pytest

import checks
from oracle import cpu_path
from oracle.cpu_path import canon_rows
from sparseconvnet_amd import synthetic

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def make():
    import torch
    assert torch.cuda.is_available()
    from hip_path import HipPath
    return lambda dim: HipPath(dim)


@pytest.mark.parametrize("dim,size", [(1, 3), (2, 3), (3, 3), (3, 2), (2, (3, 1)), (4, 3)])
def test_conv_backward(make, dim, size):
    checks.check_conv_backward(make, dim, size, seed=30 + dim, spatial=8 if dim < 4 else 5, bias=(dim != 2))


@pytest.mark.parametrize("dim,size,stride", [(3, 2, 2), (3, 3, 2), (2, 3, 2), (2, 2, 2), (1, 3, 2), (2, (3, 2), (2, 1))])
def test_strided_backward(make, dim, size, stride):
    checks.check_strided_backward(make, dim, size, stride, seed=40 + dim)


@pytest.mark.parametrize("dim", [1, 2, 3])
@pytest.mark.parametrize("thin", [1, 3, 4])
def test_thin_input_weight_gradient(make, dim, thin):
    """One to four channels on the gathered side: the weight-gradient kernel that packs several taps
    into an MFMA's rows, for filters of 3, 9 and 27 taps (submanifold), 2^dim taps from either
    side (strided: the input has the thin side; transposed: the coarse level has it) and ragged
    site counts, against torch.autograd through the dense convolutions."""
    checks.check_conv_backward(make, dim, 3, seed=130 + 10 * dim + thin, spatial=9, n=333, cin=thin, cout=20)
    checks.check_conv_backward(make, dim, 3, seed=230 + 10 * dim + thin, spatial=9, n=17, cin=thin, cout=32, bias=False)
    checks.check_strided_backward(make, dim, 2, 2, seed=330 + 10 * dim + thin, n=210, cin=thin, cout=9, pools=False)
    checks.check_strided_backward(make, dim, 2, 2, seed=430 + 10 * dim + thin, n=210, cin=24, cout=thin, pools=False)


def test_bn_train(make):
    checks.check_bn_train(make, seed=50)
    checks.check_bn_train(make, seed=51, n=5000, C=96)


def test_bn_train_full_size(make):
    """1,000,000 rows: every workgroup of the column-sum passes has work, the partial sums go
    through all sixteen wavefronts of the finishing kernels."""
    checks.check_bn_train(make, seed=52, n=1000000, C=32)


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
def test_io_backward(make, mode):
    checks.check_io_backward(make, 3, mode, seed=60 + mode)
    checks.check_bl_backward(make, 2, mode, seed=65 + mode)


def test_misc_backward(make):
    checks.check_misc_backward(make, seed=70)


@pytest.mark.parametrize("cin,cout,groups", [(3, 32, 1), (32, 32, 1), (16, 16, 1), (64, 64, 1), (96, 128, 1),
                                             (128, 160, 1), (256, 256, 1), (30, 50, 1), (8, 12, 2), (64, 32, 1),
                                             (320, 160, 1), (40, 288, 1), (96, 96, 1), (144, 48, 1), (192, 96, 1),
                                             (1, 16, 1), (4, 32, 1), (3, 20, 1)])
def test_conv_gradients_vs_oracle(oracle_built, cin, cout, groups):
    """Submanifold, strided and transposed convolution gradients on a 20,000-site room scene
    against the oracle, over the channel ranges of every forward kernel family (the input
    gradient runs through them) and of the weight-gradient kernel's tiles."""
    from hip_path import HipPath
    g, o = HipPath(3), cpu_path.CpuPath(3, "oracle")
    coords = synthetic.room_scene(seed=4200, target=20000, spatial=126, duplicate_fraction=0.0)
    rng = np.random.default_rng(cin * 1000 + cout)
    x = rng.normal(size=(len(coords), cin)).astype(np.float32)
    for p in (g, o):
        assert p.input_layer(126, coords, 0, 3) == len(coords)
        p.strided_rules(126, 63, 2, 2)
    lg, lo = g.spatial_locations(63), o.spatial_locations(63)
    rg, ro = canon_rows(lg), canon_rows(lo)

    def w(k, a, b):
        return (rng.normal(size=(k, groups, a // groups, b // groups)) * (2.0 / (a * k)) ** 0.5).astype(np.float32)
    w_s, w_d, w_u = w(27, cin, cout), w(8, cin, cout), w(8, cout, cin)
    d_y = rng.normal(size=(len(coords), cout)).astype(np.float32)
    got, want = g.subm_conv_bwd(126, 3, x, d_y, w_s, True), o.subm_conv_bwd(126, 3, x, d_y, w_s, True)
    for a, b, what in zip(got, want, ("d_input", "d_weight", "d_bias")):
        checks.assert_close(a, b, "submanifold " + what)
    # strided: the coarse level's rows are numbered differently on the two sides
    d_c = rng.normal(size=(len(lo), cout)).astype(np.float32)
    d_cg = np.empty_like(d_c)
    d_cg[rg] = d_c[ro]
    got, want = g.conv_bwd(126, 63, 2, 2, x, d_cg, w_d, True), o.conv_bwd(126, 63, 2, 2, x, d_c, w_d, True)
    for a, b, what in zip(got, want, ("d_input", "d_weight", "d_bias")):
        checks.assert_close(a, b, "strided " + what)
    xc = rng.normal(size=(len(lo), cout)).astype(np.float32)
    xg = np.empty_like(xc)
    xg[rg] = xc[ro]
    d_f = rng.normal(size=(len(coords), cin)).astype(np.float32)
    got, want = g.deconv_bwd(63, 126, 2, 2, xg, d_f, w_u, True), o.deconv_bwd(63, 126, 2, 2, xc, d_f, w_u, True)
    checks.assert_close(got[0][rg], want[0][ro], "transposed d_input")
    checks.assert_close(got[1], want[1], "transposed d_weight")
    checks.assert_close(got[2], want[2], "transposed d_bias")


@pytest.mark.parametrize("cin,cout", [(3, 32), (32, 32), (48, 64)])
def test_weight_gradient_over_many_blocks(oracle_built, cin, cout):
    """150,000 sites: more blocks of positions than the narrow layers' weight-gradient kernel has
    workgroups, so that each of them takes several turns."""
    from hip_path import HipPath
    g, o = HipPath(3), cpu_path.CpuPath(3, "oracle")
    coords = synthetic.room_scene(seed=4400, target=150000, spatial=400, duplicate_fraction=0.0)
    rng = np.random.default_rng(cin * 77 + cout)
    x = rng.normal(size=(len(coords), cin)).astype(np.float32)
    d_y = rng.normal(size=(len(coords), cout)).astype(np.float32)
    w = (rng.normal(size=(27, 1, cin, cout)) * (2.0 / (cin * 27)) ** 0.5).astype(np.float32)
    for p in (g, o):
        assert p.input_layer(400, coords, 0, 3) == len(coords)
    got, want = g.subm_conv_bwd(400, 3, x, d_y, w, True), o.subm_conv_bwd(400, 3, x, d_y, w, True)
    for a, b, what in zip(got, want, ("d_input", "d_weight", "d_bias")):
        checks.assert_close(a, b, "submanifold " + what)


def test_full_size_gradient_identities():
    """The bench scene at its full size (1,000,000 sites), where the oracle takes too long: the
    convolution is bilinear in (input, weights), so for any d_y
        <d_y, conv(x, w)> = <d_input, x> = <d_weight, w>   and   d_bias = column sums of d_y.
    A dropped tap, a share of positions counted twice or not at all, or a transposed operand breaks
    one of the equalities.  Inner products in float64 on the host; 2e-4 relative (fp32 sums of
    10^7..10^9 products on the GPU side)."""
    from hip_path import HipPath
    g = HipPath(3)
    coords = synthetic.room_scene(seed=3000, target=1000000, spatial=4096)
    n = len(coords)
    assert g.input_layer(4096, coords, 0, 0) == n
    rng = np.random.default_rng(31)
    for cin, cout in ((3, 32), (32, 32), (64, 64), (128, 128)):
        x = rng.normal(size=(n, cin)).astype(np.float32)
        d_y = rng.normal(size=(n, cout)).astype(np.float32)
        w = (rng.normal(size=(27, 1, cin, cout)) * (2.0 / (cin * 27)) ** 0.5).astype(np.float32)
        y, _ = g.subm_conv(4096, 3, x, w)
        d_x, d_w, d_b = g.subm_conv_bwd(4096, 3, x, d_y, w, True)
        dot = lambda a, b: float(np.einsum("ij,ij->", a.reshape(len(a), -1), b.reshape(len(b), -1), dtype=np.float64))
        ref = dot(d_y, y)
        scale = np.sqrt(dot(d_y, d_y) * dot(y, y))  # the size a sum of that many products could have
        assert abs(dot(d_x, x) - ref) <= 2e-4 * scale, (cin, cout, "d_input", dot(d_x, x), ref)
        assert abs(dot(d_w, w) - ref) <= 2e-4 * scale, (cin, cout, "d_weight", dot(d_w, w), ref)
        checks.assert_close(d_b, d_y.sum(0, dtype=np.float64).astype(np.float32), "d_bias at 1 M sites")
        # the weight gradient of one tap by hand: centre tap pairs every site with itself
        want = (x.astype(np.float64).T @ d_y.astype(np.float64)).astype(np.float32)
        checks.assert_close(d_w[13, 0], want, "centre-tap d_weight at 1 M sites")
    # the same identities for the 2^3 / stride-2 convolution and its transpose between 4096^3 and 2048^3
    g.strided_rules(4096, 2048, 2, 2)
    n_c = len(g.spatial_locations(2048))
    for kind, fwd, bwd, rows_in, rows_out in (("strided", g.conv, g.conv_bwd, n, n_c), ("transposed", g.deconv, g.deconv_bwd, n_c, n)):
        sizes = (4096, 2048, 2, 2) if kind == "strided" else (2048, 4096, 2, 2)
        x = rng.normal(size=(rows_in, 32)).astype(np.float32)
        d_y = rng.normal(size=(rows_out, 64)).astype(np.float32)
        w = (rng.normal(size=(8, 1, 32, 64)) * 0.1).astype(np.float32)
        y, _ = fwd(*sizes, x, w)
        d_x, d_w, d_b = bwd(*sizes, x, d_y, w, True)
        ref = dot(d_y, y)
        scale = np.sqrt(dot(d_y, d_y) * dot(y, y))
        assert abs(dot(d_x, x) - ref) <= 2e-4 * scale, (kind, "d_input", dot(d_x, x), ref)
        assert abs(dot(d_w, w) - ref) <= 2e-4 * scale, (kind, "d_weight", dot(d_w, w), ref)
        checks.assert_close(d_b, d_y.sum(0, dtype=np.float64).astype(np.float32), kind + " d_bias at 1 M sites")


def test_full_size_linear_ops_are_adjoint():
    """The bench's U-Net scene (1,300,000 points, 1,000,000 sites): every linear operator's backward
    pass is its transpose, <d_out, A f> = <A^T d_out, f> - input layer (mean of the points of a
    site), output layer, average pooling, unpooling, ActivePooling, sparse to dense at a coarse
    level; max pooling hands every gradient to the row that held the maximum, so the gradients
    of the outputs above zero all arrive and nothing else does."""
    from hip_path import HipPath
    g = HipPath(3)
    coords = synthetic.room_scene(seed=5000, target=1000000, spatial=4096, duplicate_fraction=0.3)
    n_sites = g.input_layer(4096, coords, 0, 4)
    assert len(coords) > 1200000 and 900000 < n_sites < len(coords)
    rng = np.random.default_rng(53)
    dot = lambda a, b: float(np.einsum("i,i->", a.reshape(-1), b.reshape(-1), dtype=np.float64))

    def adjoint(what, f, y, d_out, d_in):
        ref, got = dot(d_out, y), dot(d_in, f)
        assert abs(got - ref) <= 2e-4 * np.sqrt(dot(d_out, d_out) * dot(y, y)), (what, got, ref)

    f = rng.normal(size=(len(coords), 8)).astype(np.float32)
    x = g.input_fwd(f)
    assert x.shape == (n_sites, 8)
    d = rng.normal(size=x.shape).astype(np.float32)
    adjoint("input layer", f, x, d, g.input_bwd(d))
    back = g.output_fwd(x)
    d = rng.normal(size=back.shape).astype(np.float32)
    adjoint("output layer", x, back, d, g.output_bwd(d))
    g.strided_rules(4096, 2047, 3, 2)
    n_c = g.nactive(2047)
    avg = g.avgpool(4096, 2047, 3, 2, x)
    d = rng.normal(size=avg.shape).astype(np.float32)
    adjoint("average pooling", x, avg, d, g.avgpool_bwd(4096, 2047, 3, 2, 8, d))
    c = rng.normal(size=(n_c, 8)).astype(np.float32)
    up = g.unpool(2047, 4096, 3, 2, c)
    d = rng.normal(size=up.shape).astype(np.float32)
    adjoint("unpooling", c, up, d, g.unpool_bwd(2047, 4096, 3, 2, 8, d))
    mp = g.maxpool(4096, 2047, 3, 2, x)
    d = rng.normal(size=mp.shape).astype(np.float32)
    d_x = g.maxpool_bwd(4096, 2047, 3, 2, x, mp, d)
    want = np.where(mp > 0, d, 0).sum(0, dtype=np.float64)
    checks.assert_close(d_x.sum(0, dtype=np.float64), want, "max pooling: gradients that arrive")
    assert ((d_x != 0) <= (x > 0)).all()  # only a positive input can have been a maximum above zero
    ap = g.active_pooling(4096, x, True)
    d = rng.normal(size=ap.shape).astype(np.float32)
    adjoint("ActivePooling", x, ap, d, g.active_pooling_bwd(4096, d, True))
    # sparse to dense at 64^3 (dense blocks of 4096^3 do not exist): five more halvings
    size = 2047
    while size > 63:
        g.strided_rules(size, size // 2, 3, 2)
        size //= 2
    c = rng.normal(size=(g.nactive(size), 8)).astype(np.float32)
    dense = g.s2d(size, c)
    d = rng.normal(size=dense.shape).astype(np.float32)
    adjoint("sparse to dense", c, dense, d, g.s2d_bwd(size, d))


def test_pooling_and_nin_gradients_vs_oracle(oracle_built):
    from hip_path import HipPath
    g, o = HipPath(3), cpu_path.CpuPath(3, "oracle")
    coords = synthetic.room_scene(seed=4300, target=30000, spatial=127, duplicate_fraction=0.2)
    rng = np.random.default_rng(43)
    f = rng.normal(size=(len(coords), 32)).astype(np.float32)
    res = []
    for p in (g, o):
        p.input_layer(127, coords, 0, 4)
        x = p.input_fwd(f)
        p.strided_rules(127, 63, 3, 2)
        l1 = p.spatial_locations(63)
        r1 = canon_rows(l1)
        mp = p.maxpool(127, 63, 3, 2, x)
        d = np.empty_like(mp)
        d[r1] = np.random.default_rng(44).normal(size=mp.shape).astype(np.float32)
        res.append(dict(x=x, mp=mp[r1], d_max=p.maxpool_bwd(127, 63, 3, 2, x, mp, d),
                        d_avg=p.avgpool_bwd(127, 63, 3, 2, 32, d), d_avg4=p.avgpool_bwd(127, 63, 3, 2, 36, d, 4),
                        d_in=p.input_bwd(x), d_outl=p.output_bwd(f)))
        up_d = np.random.default_rng(45).normal(size=(len(x), 32)).astype(np.float32)
        res[-1]["d_un"] = p.unpool_bwd(63, 127, 3, 2, 32, up_d)[r1]
    for k in res[0]:
        checks.assert_close(res[0][k], res[1][k], k)
    for rows, cin, cout in ((70000, 64, 32), (5000, 256, 256), (777, 33, 17), (9001, 3, 32), (1, 4, 16), (500, 1, 20),
                            (4000, 96, 48)):
        a = rng.normal(size=(rows, cin)).astype(np.float32)
        w = (rng.normal(size=(cin, cout)) * 0.1).astype(np.float32)
        d = rng.normal(size=(rows, cout)).astype(np.float32)
        for u, v, what in zip(g.nin_bwd(a, d, w, True), o.nin_bwd(a, d, w, True), ("d_input", "d_weight", "d_bias")):
            checks.assert_close(u, v, "network in network %s %dx%d" % (what, cin, cout))
