"""Parity of the HIP library, called through its C ABI, with the independent statements of
tests/checks.py, with the golden fixtures written by the compiled reference, and with the
CPU oracle on the same seeded inputs.  Rulebooks bit-exact as canonically sorted
(offset, in-site, out-site) sets; features within 1e-4 relative / 1e-5 absolute (fp32)."""
import numpy as np
import pytest

import checks
from oracle import cpu_path
from oracle.cpu_path import canon_rows, canon_rules
from sparseconvnet_amd import synthetic

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def make():
    import torch
    assert torch.cuda.is_available()
    from hip_path import HipPath
    return lambda dim: HipPath(dim)


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("dim", [2, 3])
def test_input_layer(make, dim, mode):
    checks.check_input_layer(make, dim, mode, seed=10 * dim + mode)


@pytest.fixture(scope="module")
def make_host(make):
    """The same library with the coordinates handed over in host memory, as the reference's
    InputLayer receives them (scn_md_input_layer_host)."""
    def factory(dim):
        p = make(dim)
        p.host_coords = True
        return p
    return factory


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("dim", [1, 3])
def test_input_layer_from_host_coordinates(make_host, dim, mode):
    checks.check_input_layer(make_host, dim, mode, seed=10 * dim + mode)
    if mode == 4:
        checks.check_input_layer(make_host, dim, mode, seed=7, with_batch_col=False)
        checks.check_mode0_repeated_points(make_host, dim, seed=40 + dim)


def test_host_coordinates_wide_values_and_sizes(make, make_host):
    """Host coordinates are narrowed to int16 on their way to the device where the grid allows it:
    sample indices beyond int16, grids beyond int16 and inputs of several chunks give the level
    the device path gives; values outside the grid are still refused."""
    from sparseconvnet_amd._lib import ScnError
    rng = np.random.default_rng(77)
    cases = []
    c = rng.integers(0, 50, (3000, 4)).astype(np.int64)
    c[:, 3] = rng.integers(0, 3, 3000) * 20000  # sample indices 0, 20000, 40000: the last needs int32
    cases.append((50, c))
    c = rng.integers(0, 100000, (5000, 3)).astype(np.int64)  # a grid beyond int16, no sample column
    cases.append((100000, c))
    c = rng.integers(0, 300, (1500000, 4)).astype(np.int64)   # several chunks, many repeated points
    c[:, 3] = rng.integers(0, 2, len(c))
    cases.append((300, c))
    for spatial, coords in cases:
        a, b = make(3), make_host(3)
        na, nb = a.input_layer(spatial, coords, 0, 4), b.input_layer(spatial, coords, 0, 4)
        assert na == nb > 0
        assert (a.spatial_locations(spatial) == b.spatial_locations(spatial)).all()
        f = rng.normal(size=(len(coords), 2)).astype(np.float32)
        assert (a.input_fwd(f) == b.input_fwd(f)).all()
    p = make_host(3)
    for bad in ([[1, 2, 70000, 0]], [[1, -40000, 3, 0]], [[1, 2, 3, -1]], [[1 << 40, 2, 3, 0]]):
        with pytest.raises(ScnError):
            p.input_layer(64, np.array(bad, np.int64), 0, 3)
        from sparseconvnet_amd import _lib
        _lib.check(_lib.lib().scn_md_clear(p.h))
    assert p.input_layer(64, np.array([[1, 2, 3, 0], [1, 2, 3, 0]], np.int64), 0, 3) == 1


def test_input_layer_no_batch_column(make):
    checks.check_input_layer(make, 3, 4, seed=5, with_batch_col=False)
    checks.check_input_layer(make, 2, 0, seed=6, with_batch_col=False)


@pytest.mark.parametrize("dim", [1, 2, 3])
def test_input_layer_mode0_repeated_points(make, dim):
    checks.check_mode0_repeated_points(make, dim, seed=40 + dim)
    checks.check_mode0_repeated_points(make, dim, seed=50 + dim, spatial=8)
    if dim == 3:  # many workgroups, MFMA convolution kernel
        checks.check_mode0_repeated_points(make, dim, seed=44, n=20000, spatial=48, cin=16, cout=16)
        # an odd grid: the 3 / stride-2 rulebook with its candidates compacted (160 k slots)
        checks.check_mode0_repeated_points(make, dim, seed=45, n=20000, spatial=49, cin=8, cout=8)


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("dim", [2, 3])
def test_bl_input_layer(make, dim, mode):
    checks.check_bl_input_layer(make, dim, mode, seed=20 * dim + mode)


def test_bl_input_layer_edge_cases(make):
    checks.check_bl_input_layer(make, 3, 3, seed=1, empties=False)
    checks.check_bl_input_layer(make, 1, 4, seed=2, batch=1, length=300, spatial=40)
    checks.check_bl_input_layer(make, 2, 1, seed=3, batch=5, length=1)


@pytest.mark.parametrize("dim", [1, 2, 3])
def test_input_batch(make, dim):
    checks.check_input_batch(make, dim, seed=70 + dim)


@pytest.mark.parametrize("dim,size,spatial", [(3, 2, 24), (3, 3, 23), (2, 2, (24, 12)), (2, 3, 47), (1, 2, 40)])
def test_generate_rulebooks(make, dim, size, spatial):
    checks.check_generate_rulebooks(make, dim, size, spatial, seed=80 + dim + size)


@pytest.mark.parametrize("dim", [5, 6])
def test_high_dimensions(make, dim):
    # sparseconvnet_cpu.cpp:14-20 instantiates dimensions 1..6
    checks.check_input_layer(make, dim, 4, seed=90 + dim, spatial=3, n=250)
    checks.check_submanifold(make, dim, 3 if dim == 5 else (3, 1, 3, 1, 3, 1), seed=91 + dim, spatial=3, n=150)
    checks.check_strided(make, dim, 2, 2, seed=92 + dim, out_spatial=2, n=150)
    checks.check_s2d(make, dim, seed=93 + dim, spatial=3, n=80)
    checks.check_input_batch(make, dim, seed=94 + dim, spatial=4)


@pytest.mark.parametrize("dim,size", [(1, 3), (2, 3), (3, 3), (2, (3, 1)), (3, (1, 3, 5)), (3, 2),
                                      (4, 3)])
def test_submanifold(make, dim, size):
    checks.check_submanifold(make, dim, size, seed=7 + dim, spatial=8 if dim < 4 else 5,
                             n=200 if dim < 4 else 250, bias=(dim == 2))


@pytest.mark.parametrize("dim,size,stride", [(3, 2, 2), (3, 3, 2), (2, 3, 2), (2, 2, 2), (1, 3, 2),
                                             (2, (3, 2), (2, 1)), (3, 4, 2), (2, 2, 3), (3, 3, 1)])
def test_strided(make, dim, size, stride):
    checks.check_strided(make, dim, size, stride, seed=3 + dim, bias=(dim == 2))


@pytest.mark.parametrize("dim,mode,cin,cout", [(3, 4, 64, 32), (3, 4, 64, 24), (3, 4, 64, 16), (3, 4, 32, 32), (3, 4, 32, 16),
                                               (3, 4, 32, 9), (2, 4, 64, 32), (1, 4, 32, 16), (3, 0, 64, 32), (2, 0, 32, 20)])
def test_deconvolution_with_all_taps_resident(make, dim, mode, cin, cout):
    """Transposed convolution of a 2^3 / stride-2 rulebook at the plane counts whose weights of all
    eight taps fit LDS (the kernel that reads the one rule of every fine position instead of the
    table's columns): against the rules applied by hand, with a bias, and with a batch norm + leaky
    ReLU behind it; in one to three dimensions (2, 4, 8 taps), and on a level with repeated points
    (input-layer mode 0: the rows a later point of their site shadows have no rule and get the bias)."""
    rng = np.random.default_rng(cin + cout + dim)
    n, spatial = 3000, {1: 4000, 2: 120, 3: 40}[dim]
    pts = np.concatenate([rng.integers(0, spatial, (n, dim)), rng.integers(0, 3, (n, 1))], 1)
    if mode == 0:
        pts = np.concatenate([pts, pts[rng.integers(0, n, n // 4)]], 0)  # a quarter of the points once more
    else:
        pts = np.unique(pts, axis=0)
    pts = pts[rng.permutation(len(pts))].astype(np.int64)
    p = make(dim)
    assert p.input_layer(spatial, pts, 0, mode) == len(pts)
    rules = p.strided_rules(spatial, spatial // 2, 2, 2)
    n_coarse = p.nactive(spatial // 2)
    y = rng.normal(size=(n_coarse, cin)).astype(np.float32)
    w = (rng.normal(size=(2 ** dim, 1, cin, cout)) * 0.2).astype(np.float32)
    b = rng.normal(size=cout).astype(np.float32)
    want = np.zeros((len(pts), cout), np.float64)
    for k, r in enumerate(rules):  # the rulebook of the convolution, read backwards
        want[r[:, 0]] += y[r[:, 1]].astype(np.float64) @ w[k, 0].astype(np.float64)
    z, macs = p.deconv(spatial // 2, spatial, 2, 2, y, w)
    assert macs == sum(len(r) for r in rules) * cin * cout
    checks.assert_close(z, want, "transposed convolution")
    zb, _ = p.deconv(spatial // 2, spatial, 2, 2, y, w, b)
    checks.assert_close(zb, want + b, "transposed convolution with bias")
    bn = dict(mean=rng.normal(size=cout).astype(np.float32), var=rng.uniform(0.5, 1.5, cout).astype(np.float32),
              weight=rng.uniform(0.5, 1.5, cout).astype(np.float32), bias=rng.normal(size=cout).astype(np.float32),
              eps=1e-4, leakiness=0.25)
    zp, _ = p.deconv(spatial // 2, spatial, 2, 2, y, w, b, post=bn)
    sc = bn["weight"] / np.sqrt(bn["var"] + np.float32(1e-4))
    v = (want + b) * sc + (bn["bias"] - bn["mean"] * sc)
    checks.assert_close(zp, np.where(v > 0, v, 0.25 * v), "transposed convolution + batch norm + leaky ReLU")


def test_bn(make):
    checks.check_bn(make, seed=1)
    checks.check_bn(make, seed=2, n=1000, C=32)


def test_nin(make):
    checks.check_nin(make, seed=4)
    # every convolution kernel family: few / many output planes, wide inputs, odd plane counts
    checks.check_nin(make, seed=5, shapes=((5000, 64, 32), (5000, 32, 64), (3000, 96, 160), (2000, 256, 256),
                                           (70000, 64, 32), (777, 33, 17), (4000, 3, 32), (1500, 448, 224)))
    # the shapes whose whole weight matrix stays in LDS, at ragged row counts
    checks.check_nin(make, seed=6, shapes=((1, 64, 32), (63, 64, 16), (4097, 32, 32), (33333, 32, 16), (9000, 64, 24),
                                           (300001, 64, 32), (5000, 32, 8)))


@pytest.mark.parametrize("dim", [1, 2, 3])
def test_s2d(make, dim):
    checks.check_s2d(make, dim, seed=2 + dim)


@pytest.mark.parametrize("dim", [1, 2, 3, 4])
def test_active_pooling(make, dim):
    checks.check_active_pooling(make, dim, seed=70 + dim)


@pytest.mark.parametrize("planes,n", [(96, 3000), (64, 20000), (7, 5000)])
def test_active_pooling_wide(make, planes, n):
    """More planes than one 64-plane tile of the kernels, plane counts that do and do not allow
    16-byte loads, and samples of thousands of sites (several chunks of rows per sample)."""
    checks.check_active_pooling(make, 3, seed=90 + planes, spatial=40, n=n, batch=3, C=planes)


def test_level_replacement(make):
    checks.check_level_replacement(make)


def test_special_values(make):
    checks.check_special_values(make)


def test_empty(make):
    checks.check_empty(make)


def test_golden(make, tmp_path):
    from test_golden import compare_with_golden, make_golden
    for name in sorted(make_golden.FIXTURES):
        compare_with_golden(name, make, tmp_path)


def _both(dim, oracle_built):
    from hip_path import HipPath
    return HipPath(dim), cpu_path.CpuPath(dim, "oracle")


@pytest.mark.parametrize("cin,cout,groups", [(16, 16, 1), (3, 32, 1), (8, 12, 2), (32, 32, 1), (64, 64, 1)])
def test_config1_vs_oracle(oracle_built, cin, cout, groups):
    """Configuration 1 (batch 2, 128^3, ~40k sites per sample, 3^3 submanifold convolution)."""
    g, o = _both(3, oracle_built)
    coords = synthetic.config1()
    rng = np.random.default_rng(1)
    x = rng.normal(size=(len(coords), cin)).astype(np.float32)
    w = (rng.normal(size=(27, groups, cin // groups, cout // groups)) * (2.0 / (cin * 27)) ** 0.5).astype(
        np.float32)
    for p in (g, o):
        assert p.input_layer(128, coords, 0, 0) == len(coords)
    lg, lo = g.spatial_locations(128), o.spatial_locations(128)
    assert (lg == lo).all() and (lg == coords).all()
    rg, ro = g.submanifold_rules(128, 3), o.submanifold_rules(128, 3)
    assert (canon_rules(rg, lg, lg) == canon_rules(ro, lo, lo)).all()
    yg, mg = g.subm_conv(128, 3, x, w)
    yo, mo = o.subm_conv(128, 3, x, w)
    assert mg == mo
    checks.assert_close(yg, yo, "config 1 conv")


def test_strided_tree_vs_oracle(oracle_built):
    """Configuration 4's tree at 254^3 with 60k points, duplicates merged by mode 4."""
    g, o = _both(3, oracle_built)
    coords = synthetic.room_scene(seed=4000, target=60000, spatial=254, duplicate_fraction=0.3)
    rng = np.random.default_rng(4)
    f = rng.uniform(-1, 1, size=(len(coords), 32)).astype(np.float32)
    w1 = (rng.normal(size=(8, 1, 32, 64)) * 0.1).astype(np.float32)
    w2 = (rng.normal(size=(8, 1, 64, 32)) * 0.1).astype(np.float32)
    res = []
    for p in (g, o):
        p.input_layer(254, coords, 0, 4)
        l0 = p.spatial_locations(254)
        x = p.input_fwd(f)
        r1 = p.strided_rules(254, 127, 2, 2)
        l1 = p.spatial_locations(127)
        h, m1 = p.conv(254, 127, 2, 2, x, w1)
        r2 = p.strided_rules(127, 63, 3, 2)
        l2 = p.spatial_locations(63)
        mp = p.maxpool(127, 63, 3, 2, h)
        u, m2 = p.deconv(127, 254, 2, 2, h, w2)
        res.append(dict(l0=l0, x=x, r1=canon_rules(r1, l0, l1), l1=l1[canon_rows(l1)], h=h[canon_rows(l1)],
                        m1=m1, r2=canon_rules(r2, l1, l2), mp=mp[canon_rows(l2)], u=u, m2=m2,
                        back=p.output_fwd(u)))
    a, b = res
    for k in ("l0", "r1", "l1", "r2"):
        assert a[k].shape == b[k].shape and (a[k] == b[k]).all(), k
    assert a["m1"] == b["m1"] and a["m2"] == b["m2"]
    for k in ("x", "h", "mp", "u", "back"):
        checks.assert_close(a[k], b[k], k)


@pytest.mark.parametrize("cin,cout,groups", [(3, 32, 1), (32, 32, 1), (40, 16, 1), (48, 64, 1), (64, 96, 1),
                                             (96, 128, 1), (128, 160, 1), (30, 50, 1), (64, 32, 1), (8, 12, 2),
                                             (48, 320, 1)])
def test_fused_bn_conv_vs_oracle(oracle_built, cin, cout, groups):
    """The fused entry point (eval batch norm + leaky ReLU in front of the convolution applied
    in its gather, the one behind it applied to its stores) against the oracle's separate
    passes, over every convolution kernel's channel range, for the submanifold, strided and
    transposed convolutions."""
    g, o = _both(3, oracle_built)
    coords = synthetic.room_scene(seed=4100, target=20000, spatial=126, duplicate_fraction=0.0)
    rng = np.random.default_rng(cin * 1000 + cout)
    x = rng.normal(size=(len(coords), cin)).astype(np.float32)

    def bn_of(planes, leak, affine=True):
        return dict(mean=rng.normal(size=planes).astype(np.float32),
                    var=rng.uniform(0.5, 1.5, planes).astype(np.float32),
                    weight=rng.uniform(0.5, 1.5, planes).astype(np.float32) if affine else None,
                    bias=rng.normal(size=planes).astype(np.float32) if affine else None, eps=1e-4, leakiness=leak)

    def apply(p, bn, v):
        return p.bn_eval(v, bn["mean"], bn["var"], bn["weight"], bn["bias"], bn["eps"], bn["leakiness"])

    def w(k, a, b):
        return (rng.normal(size=(k, groups, a // groups, b // groups)) * (2.0 / (a * k)) ** 0.5).astype(np.float32)
    pre, post, post_leaky = bn_of(cin, 0.0), bn_of(cout, 0.0), bn_of(cout, 0.333, affine=False)
    w_s, w_d, w_u = w(27, cin, cout), w(8, cin, cout), w(8, cin, cout)
    bias = rng.normal(size=cout).astype(np.float32)
    for p in (g, o):
        assert p.input_layer(126, coords, 0, 3) == len(coords)
        p.strided_rules(126, 63, 2, 2)
    lg, lo = g.spatial_locations(63), o.spatial_locations(63)
    xn = apply(o, pre, x)
    # batch norm in front and behind
    got, _ = g.subm_conv(126, 3, x, w_s, bias, bn=pre, post=post)
    want = apply(o, post, o.subm_conv(126, 3, xn, w_s, bias)[0])
    checks.assert_close(got, want, "bn + submanifold convolution + bn")
    # only behind
    got, _ = g.subm_conv(126, 3, x, w_s, None, post=post_leaky)
    want = apply(o, post_leaky, o.subm_conv(126, 3, x, w_s, None)[0])
    checks.assert_close(got, want, "submanifold convolution + bn")
    # only in front
    got, m1 = g.conv(126, 63, 2, 2, x, w_d, None, bn=pre)
    want, m2 = o.conv(126, 63, 2, 2, xn, w_d, None)
    assert m1 == m2
    checks.assert_close(got[canon_rows(lg)], want[canon_rows(lo)], "bn + strided convolution")
    got, _ = g.conv(126, 63, 2, 2, x, w_d, bias, post=post)
    want = apply(o, post, o.conv(126, 63, 2, 2, x, w_d, bias)[0])
    checks.assert_close(got[canon_rows(lg)], want[canon_rows(lo)], "strided convolution + bn")
    # transposed convolution: rows of the 63^3 level in, rows of the 126^3 level out
    xc = rng.normal(size=(len(lo), cin)).astype(np.float32)
    xg = np.empty_like(xc)
    xg[canon_rows(lg)] = xc[canon_rows(lo)]  # the same site gets the same row of values
    leaky = bn_of(cin, 0.333, affine=False)
    got, _ = g.deconv(63, 126, 2, 2, xg, w_u, bias, bn=leaky, post=post)
    want = apply(o, post, o.deconv(63, 126, 2, 2, apply(o, leaky, xc), w_u, bias)[0])
    checks.assert_close(got, want, "bn + transposed convolution + bn")


def _neighbour_counts(coords, spatial):
    """Per site and tap: is the neighbour active?  Independent of oracle and library: sorted
    linear indices and a binary search (numpy)."""
    c = coords[:, :3].astype(np.int64)
    lin = ((coords[:, 3].astype(np.int64) * spatial + c[:, 0]) * spatial + c[:, 1]) * spatial + c[:, 2]
    order = np.argsort(lin)
    s = lin[order]
    present = np.zeros((27, len(c)), bool)
    k = 0
    for dx in (-1, 0, 1):
        for dy in (-1, 0, 1):
            for dz in (-1, 0, 1):
                q = lin + (dx * spatial + dy) * spatial + dz
                ok = ((c[:, 0] + dx >= 0) & (c[:, 0] + dx < spatial) & (c[:, 1] + dy >= 0) & (c[:, 1] + dy < spatial)
                      & (c[:, 2] + dz >= 0) & (c[:, 2] + dz < spatial))
                i = np.minimum(np.searchsorted(s, q), len(s) - 1)
                present[k] = ok & (s[i] == q)
                k += 1
    return present


@pytest.mark.parametrize("cin,cout", [(32, 32), (32, 16), (64, 64), (64, 32), (128, 128), (96, 160), (256, 256), (128, 32)])
def test_bf16_path_vs_oracle(oracle_built, cin, cout):
    """The optional bf16-operand path: submanifold convolution (with and without a batch norm
    in front), strided convolution and deconvolution against the fp32 oracle, every element within
    1e-2 relative + 4e-3 of the largest output; the fp32 path on the same handle stays within its own
    tolerance."""
    hp, op = _both(3, oracle_built)
    hp.set_bf16(True)
    rng = np.random.default_rng(cin * 7 + cout)
    coords = synthetic.scene_batch(seed=8000 + cin, batch=2, target=4000, spatial=64, n_boxes=8)
    for p in (hp, op):
        p.input_layer(64, coords, 0, 3)
    x = rng.normal(size=(len(coords), cin)).astype(np.float32)
    xo, xh = op.input_fwd(x), hp.input_fwd(x)
    ro, rh = canon_rows(op.spatial_locations(64)), canon_rows(hp.spatial_locations(64))

    def close(got, want, what):
        # 1e-2 relative per element, plus an absolute term for elements that are small through
        # cancellation: operands rounded to 8 significant bits put an error of about 2e-3 of the
        # output's root mean square on every sum, whatever the sum's own size (4e-3 of the largest
        # output is a few times that).
        scale = float(np.abs(want).max())
        err = np.abs(got.astype(np.float64) - want)
        bad = err > 4e-3 * scale + 1e-2 * np.abs(want)
        assert not bad.any(), "%s: %d/%d off, max err %g against scale %g" % (what, bad.sum(), bad.size, err.max(), scale)
        assert err.max() > 0  # the reduced-precision kernels did run

    w = (rng.normal(size=(27, 1, cin, cout)) * (2.0 / (cin * 27)) ** 0.5).astype(np.float32)
    yo, _ = op.subm_conv(64, 3, xo, w)
    yh, _ = hp.subm_conv(64, 3, xh, w)
    close(yh[rh], yo[ro], "submanifold")
    bn = dict(mean=rng.normal(size=cin).astype(np.float32), var=rng.uniform(0.5, 1.5, cin).astype(np.float32),
              weight=rng.normal(size=cin).astype(np.float32), bias=rng.normal(size=cin).astype(np.float32),
              eps=1e-4, leakiness=0.0)
    xb = op.bn_eval(xo, bn["mean"], bn["var"], bn["weight"], bn["bias"], 1e-4, 0.0)
    yo, _ = op.subm_conv(64, 3, xb, w)
    yh, _ = hp.subm_conv(64, 3, xh, w, bn=bn)
    close(yh[rh], yo[ro], "batch norm + submanifold")
    w2 = (rng.normal(size=(8, 1, cin, cout)) * (2.0 / (cin * 8)) ** 0.5).astype(np.float32)
    co, _ = op.conv(64, 32, 2, 2, xo, w2)
    ch, _ = hp.conv(64, 32, 2, 2, xh, w2)
    r1o, r1h = canon_rows(op.spatial_locations(32)), canon_rows(hp.spatial_locations(32))
    close(ch[r1h], co[r1o], "strided")
    w3 = (rng.normal(size=(8, 1, cout, cin)) * (2.0 / (cout * 8)) ** 0.5).astype(np.float32)
    do, _ = op.deconv(32, 64, 2, 2, co, w3)
    dh, _ = hp.deconv(32, 64, 2, 2, co[r1o][np.argsort(r1h)], w3)
    close(dh[rh], do[ro], "transposed")
    hp.set_bf16(False)
    yo, _ = op.subm_conv(64, 3, xo, w)
    yh, _ = hp.subm_conv(64, 3, xh, w)
    checks.assert_close(yh[rh], yo[ro], "fp32 again")


def test_full_size_sweep_scene_properties():
    """Configuration 3 at its full size (one room scene of 1,000,000 sites in 4096^3, the
    bench workload), through properties that do not need the oracle to finish: the rule count
    per tap equals an independent numpy count; a convolution whose weights are all ones on a
    feature of ones returns each site's neighbour count; the centre-tap identity returns the
    input; the map is linear; fused and separate batch norm agree."""
    from hip_path import HipPath
    g = HipPath(3)
    coords = synthetic.room_scene(seed=3000, target=1000000, spatial=4096)
    assert g.input_layer(4096, coords, 0, 0) == len(coords)
    present = _neighbour_counts(coords, 4096)
    rules = g.submanifold_rules(4096, 3)
    assert [len(r) for r in rules] == present.sum(1).tolist()
    # taps are mirror images of each other: rule (i -> j) of tap k is rule (j -> i) of tap 26 - k
    for k in (0, 5, 13):
        a, b = rules[k], rules[26 - k]
        ka = np.sort(a[:, 0].astype(np.int64) * len(coords) + a[:, 1])
        kb = np.sort(b[:, 1].astype(np.int64) * len(coords) + b[:, 0])
        assert (ka == kb).all()
    n = len(coords)
    ones = np.ones((n, 1), np.float32)
    y, macs = g.subm_conv(4096, 3, ones, np.ones((27, 1, 1, 1), np.float32))
    assert macs == present.sum()
    assert (y[:, 0] == present.sum(0)).all()  # small integers: exact in fp32
    rng = np.random.default_rng(3)
    for cin, cout in ((32, 32), (64, 64), (128, 128)):
        x = rng.normal(size=(n, cin)).astype(np.float32)
        w = np.zeros((27, 1, cin, cout), np.float32)
        w[13, 0] = np.eye(cin, cout)
        y, _ = g.subm_conv(4096, 3, x, w)
        assert (y == x[:, :cout]).all()  # centre tap, identity weights: a copy
    x1, x2 = rng.normal(size=(n, 64)).astype(np.float32), rng.normal(size=(n, 64)).astype(np.float32)
    w = (rng.normal(size=(27, 1, 64, 64)) * (2.0 / (64 * 27)) ** 0.5).astype(np.float32)
    y1, y2, y12 = (g.subm_conv(4096, 3, v, w)[0] for v in (x1, x2, x1 + 2 * x2))
    checks.assert_close(y12, y1 + 2 * y2, "linearity at 1 M sites")
    # one output row recomputed by hand from the numpy neighbour table
    lin = ((coords[:, 0].astype(np.int64)) * 4096 + coords[:, 1]) * 4096 + coords[:, 2]
    order = np.argsort(lin)
    for row in (0, n // 2, n - 1):
        acc = np.zeros(64, np.float64)
        k = 0
        for dx in (-1, 0, 1):
            for dy in (-1, 0, 1):
                for dz in (-1, 0, 1):
                    if present[k, row]:
                        q = lin[row] + (dx * 4096 + dy) * 4096 + dz
                        j = order[np.searchsorted(lin[order], q)]
                        acc += x1[j].astype(np.float64) @ w[k, 0].astype(np.float64)
                    k += 1
        checks.assert_close(y1[row], acc, "row %d by hand" % row)
    bn = dict(mean=rng.normal(size=64).astype(np.float32), var=rng.uniform(0.5, 1.5, 64).astype(np.float32),
              weight=rng.uniform(0.5, 1.5, 64).astype(np.float32), bias=rng.normal(size=64).astype(np.float32),
              eps=1e-4, leakiness=0.0)
    fused, _ = g.subm_conv(4096, 3, x1, w, None, bn=bn, post=bn)
    sep = g.bn_eval(g.subm_conv(4096, 3, g.bn_eval(x1, bn["mean"], bn["var"], bn["weight"], bn["bias"], 1e-4, 0.0),
                                w)[0], bn["mean"], bn["var"], bn["weight"], bn["bias"], 1e-4, 0.0)
    checks.assert_close(fused, sep, "fused vs separate batch norm at 1 M sites")


def test_input_above_2_gib_matches_split_channels():
    """A feature matrix above 2 GiB takes the kernels' 64-bit addressing path (the buffer-load
    gathers are for smaller inputs; the reference itself overflows its int32 offsets near this
    size, CPU/Convolution.cpp:18,38).  Checked against the same convolution computed as the
    sum of two half-width convolutions, each of which is below the limit."""
    import torch
    from sparseconvnet_amd import metadata as M
    coords = synthetic.room_scene(seed=3100, target=1100000, spatial=4096)
    n = len(coords)
    md = M.Metadata(3)
    sz, three = torch.LongTensor([4096] * 3), torch.LongTensor([3] * 3)
    g = torch.Generator(device="cuda").manual_seed(31)
    md.inputLayer(sz, torch.as_tensor(coords).cuda(), torch.zeros((n, 1), device="cuda"), 0, 0)
    x = torch.randn((n, 512), device="cuda", generator=g)
    assert x.numel() * 4 > 2 ** 31
    for cout in (16, 144):  # row-owner kernel, LDS-tiled kernel
        w = torch.randn((27, 1, 512, cout), device="cuda", generator=g) * 0.02
        y, macs = md.submanifoldConvolution(sz, three, x, w, None)
        ya, _ = md.submanifoldConvolution(sz, three, x[:, :256].contiguous(), w[:, :, :256].contiguous(), None)
        yb, _ = md.submanifoldConvolution(sz, three, x[:, 256:].contiguous(), w[:, :, 256:].contiguous(), None)
        want = (ya + yb).cpu().numpy()
        checks.assert_close(y.cpu().numpy(), want, "512 -> %d above 2 GiB" % cout)
        assert np.abs(want).max() > 0.1 and macs > 0
        del y, ya, yb


def test_error_paths_leave_the_handle_usable(make):
    """Every misuse comes back as a status plus message (ScnError here), no kernel runs on bad
    operands, and the handle keeps working afterwards."""
    import ctypes as C
    import torch
    from sparseconvnet_amd import _lib
    from sparseconvnet_amd._lib import ScnError
    L = _lib.lib()
    assert L.scn_md_create(0) is None and L.scn_md_create(9) is None
    assert b"dimension" in L.scn_last_error() or len(L.scn_last_error()) > 0
    with pytest.raises(ScnError, match="null metadata handle"):
        _lib.check(L.scn_md_clear(None))
    p = make(3)
    good = np.array([[1, 2, 3, 0], [4, 5, 6, 1], [1, 2, 3, 0]], np.int64)
    for bad, what in (([[1, 2, 8, 0]], "outside"), ([[-1, 2, 3, 0]], "outside"), ([[1, 2, 3, -1]], "sample index")):
        with pytest.raises(ScnError, match=what):
            p.input_layer(8, np.array(bad, np.int64), 0, 3)
        _lib.check(L.scn_md_clear(p.h))
    with pytest.raises(ScnError, match="mode"):
        p.input_layer(8, good, 0, 7)
    _lib.check(L.scn_md_clear(p.h))
    with pytest.raises(ScnError, match="every position filled"):
        p.bl_input_layer(8, np.array([[[1, 1, 1], [-1, -1, -1]]], np.int64), 0)
    _lib.check(L.scn_md_clear(p.h))
    with pytest.raises(ScnError, match="not been built"):
        p.input_rules()
    assert p.input_layer(8, good, 0, 3) == 2
    with pytest.raises(ScnError, match="already has an input layer"):
        p.input_layer(8, good, 0, 3)
    x = np.ones((2, 4), np.float32)
    with pytest.raises(ScnError, match="kind"):
        hdr = (C.c_int64 * 3)(8, 8, 8)
        xd = torch.ones(2, 4, device="cuda")
        _lib.check(L.scn_conv_bn_fwd(p.h, 5, hdr, hdr, None, None, C.c_void_p(xd.data_ptr()), C.c_void_p(xd.data_ptr()),
                                     C.c_void_p(xd.data_ptr()), None, 4, 4, 1, None, None, None, None))
    with pytest.raises(ScnError, match="planes must equal"):
        sz = [p._s(v) for v in (8, 4, 2, 2)]
        _lib.check(L.scn_md_strided_rules(p.h, *sz, None))
        xd = torch.ones(2, 4, device="cuda")
        _lib.check(L.scn_maxpool_fwd(p.h, *sz, C.c_void_p(xd.data_ptr()), 4, C.c_void_p(xd.data_ptr()), 4, 1, None))
    with pytest.raises(ScnError, match="unknown spatial size"):
        p.s2d(5, x)
    with pytest.raises(ScnError, match="filter"):
        p.submanifold_rules(8, 0)
    # the handle still works
    y, macs = p.subm_conv(8, 3, x, np.ones((27, 1, 4, 2), np.float32))
    assert y.shape == (2, 2) and macs == 2 * 4 * 2 and (y == 4).all()


def test_failed_input_layer_leaves_no_level_behind(make):
    """A construction that fails is undone: the handle takes the next input layer without a
    scn_md_clear in between."""
    from sparseconvnet_amd._lib import ScnError
    p = make(3)
    with pytest.raises(ScnError, match="outside"):
        p.input_layer(8, np.array([[1, 2, 9, 0]], np.int64), 0, 3)
    assert p.nactive(8) == 0
    with pytest.raises(ScnError, match="not been built"):
        p.input_rules()
    good = np.array([[1, 2, 3, 0], [4, 5, 6, 1], [1, 2, 3, 0]], np.int64)
    assert p.input_layer(8, good, 0, 3) == 2
    y, macs = p.subm_conv(8, 3, np.ones((2, 4), np.float32), np.ones((27, 1, 4, 2), np.float32))
    assert (y == 4).all() and macs == 2 * 4 * 2


def test_block_cache_across_streams_and_release():
    """Handles driven from different streams hand their blocks to each other through the
    library's cache (a block freed by one stream's handle is waited for before another stream's
    handle writes it): results stay those of the single-stream run.  scn_release_cache gives the
    idle blocks back; a destroyed handle's multiply-add counts are collected without a wait at
    destruction."""
    import ctypes as C
    import torch
    from sparseconvnet_amd import _lib
    L = _lib.lib()
    coords = [torch.as_tensor(synthetic.room_scene(seed=6100 + i, target=40000, spatial=512)).cuda() for i in range(2)]
    g = torch.Generator(device="cuda").manual_seed(6)
    w = torch.randn((27, 1, 32, 32), device="cuda", generator=g) * 0.05
    xs = [torch.randn((len(c), 32), device="cuda", generator=g) for c in coords]
    sp, fs = _lib.sizes(3, 512), _lib.sizes(3, 3)

    def run(stream, i):
        with torch.cuda.stream(stream):
            sv = C.c_void_p(stream.cuda_stream)
            h = L.scn_md_create(3)
            n = C.c_int64(0)
            _lib.check(L.scn_md_input_layer(h, sp, C.c_void_p(coords[i].data_ptr()), len(coords[i]), 4, 0, 0, sv, C.byref(n)))
            y = torch.empty((n.value, 32), device="cuda")
            _lib.check(L.scn_subm_conv_fwd(h, sp, fs, C.c_void_p(xs[i].data_ptr()), C.c_void_p(y.data_ptr()),
                                           C.c_void_p(w.data_ptr()), None, 32, 32, 1, sv, None))
            L.scn_md_destroy(h)  # its blocks go back while the convolution may still be running
        return y
    torch.cuda.synchronize()
    main = torch.cuda.current_stream()
    want = [run(main, i) for i in range(2)]
    torch.cuda.synchronize()
    released = C.c_double(0)
    _lib.check(L.scn_take_released_macs(C.byref(released)))
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    got = []
    for rep in range(6):
        got.append((rep % 2, run(s1 if rep % 2 == 0 else s2, rep % 2)))
    torch.cuda.synchronize()
    for i, y in got:
        assert torch.equal(y, want[i])
    _lib.check(L.scn_take_released_macs(C.byref(released)))
    assert released.value > 0 and released.value % (32 * 32) == 0
    live, idle, peak, mallocs = (C.c_int64(0) for _ in range(4))
    _lib.check(L.scn_cache_stats(C.byref(live), C.byref(idle), C.byref(peak), C.byref(mallocs)))
    assert idle.value > 0 and peak.value >= idle.value + live.value
    _lib.check(L.scn_release_cache())
    _lib.check(L.scn_cache_stats(C.byref(live), C.byref(idle), None, None))
    assert idle.value == 0
    y = run(main, 0)
    torch.cuda.synchronize()
    assert torch.equal(y, want[0])
