"""The benchmark configurations at their full sizes, where the CPU oracle is too slow to be the
checker: properties that numpy can state independently of oracle and library (rule sets from
sorted linear indices, neighbour counts, identity taps, rows recomputed by hand, linearity)
and invariances of the path (cold == warm, samples never interact, point order).  Rule sets
bit-exact; features within 1e-4 relative / 1e-5 absolute (fp32)."""
import numpy as np
import pytest

import checks
from sparseconvnet_amd import synthetic

pytestmark = pytest.mark.gpu


def _lin(c, spatial):
    """Row-major linear index of [n, 3(+1)] coordinates (sample index, if any, in front)."""
    c = c.astype(np.int64)
    b = c[:, 3] if c.shape[1] > 3 else 0
    return ((b * spatial + c[:, 0]) * spatial + c[:, 1]) * spatial + c[:, 2]


def _present(coords, spatial):
    """present[k, i]: is the neighbour of site i at tap k (row-major 3^3 box, last coordinate
    fastest, SCN/Metadata/RectangularRegions.h:56-71) active?  nb[k, i]: its row."""
    c = coords[:, :3].astype(np.int64)
    lin = _lin(coords, spatial)
    order = np.argsort(lin)
    s = lin[order]
    present = np.zeros((27, len(c)), bool)
    nb = np.zeros((27, len(c)), np.int64)
    k = 0
    for dx in (-1, 0, 1):
        for dy in (-1, 0, 1):
            for dz in (-1, 0, 1):
                q = lin + (dx * spatial + dy) * spatial + dz
                ok = np.ones(len(c), bool)
                for d, o in enumerate((dx, dy, dz)):
                    ok &= (c[:, d] + o >= 0) & (c[:, d] + o < spatial)
                i = np.minimum(np.searchsorted(s, q), len(s) - 1)
                present[k] = ok & (s[i] == q)
                nb[k] = order[i]
                k += 1
    return present, nb


@pytest.fixture(scope="module")
def sweep_scene():
    """Configuration 3's scene with its rulebook built once for the tests below."""
    from hip_path import HipPath
    g = HipPath(3)
    coords = synthetic.room_scene(seed=3000, target=1000000, spatial=4096)
    assert g.input_layer(4096, coords, 0, 0) == len(coords)
    present, nb = _present(coords, 4096)
    return g, coords, present, nb


def test_sweep_rule_sets_are_exact_at_1m_sites(sweep_scene):
    """Every (tap, in, out) triple of the 1 M-site submanifold rulebook against the numpy
    neighbour table: the whole set, not only its size."""
    g, coords, present, nb = sweep_scene
    rules = g.submanifold_rules(4096, 3)
    n = len(coords)
    for k in range(27):
        out_rows = np.nonzero(present[k])[0]
        want = np.sort(nb[k, out_rows] * n + out_rows)
        got = np.sort(rules[k][:, 0].astype(np.int64) * n + rules[k][:, 1])
        assert got.shape == want.shape and (got == want).all(), "tap %d" % k


@pytest.mark.parametrize("cin,cout", [(3, 32), (256, 256)])
def test_sweep_ends_at_1m_sites(sweep_scene, cin, cout):
    """The two ends of the bench sweep at the bench size: 3 -> 32 (the four-channel resident
    kernel) and 256 -> 256 (the LDS-tiled kernel with buffer gathers, the kernel the headline
    roofline figure is quoted on)."""
    g, coords, present, nb = sweep_scene
    n = len(coords)
    counts = present.sum(0)
    y, macs = g.subm_conv(4096, 3, np.ones((n, cin), np.float32), np.ones((27, 1, cin, cout), np.float32))
    assert macs == float(present.sum()) * cin * cout
    assert (y == (counts * cin)[:, None]).all()  # small integers: exact in fp32
    rng = np.random.default_rng(cin)
    x1 = rng.normal(size=(n, cin)).astype(np.float32)
    w = np.zeros((27, 1, cin, cout), np.float32)
    w[13, 0] = np.eye(cin, cout)
    y, _ = g.subm_conv(4096, 3, x1, w)
    assert (y[:, :min(cin, cout)] == x1[:, :cout]).all() and (y[:, cin:] == 0).all()  # centre tap: a copy
    del y
    w = (rng.normal(size=(27, 1, cin, cout)) * (2.0 / (cin * 27)) ** 0.5).astype(np.float32)
    bias = rng.normal(size=cout).astype(np.float32)
    y1, _ = g.subm_conv(4096, 3, x1, w, bias)
    rows = [0, 1, n // 3, n // 2, n - 2, n - 1, int(np.argmax(counts)), int(np.argmin(counts))]
    for row in rows:
        acc = bias.astype(np.float64)
        for k in np.nonzero(present[:, row])[0]:
            acc = acc + x1[nb[k, row]].astype(np.float64) @ w[k, 0].astype(np.float64)
        checks.assert_close(y1[row], acc, "row %d of %d -> %d by hand" % (row, cin, cout))
    x2 = rng.normal(size=(n, cin)).astype(np.float32)
    y2, _ = g.subm_conv(4096, 3, x2, w)
    y12, _ = g.subm_conv(4096, 3, x1 + 2 * x2, w, bias)
    checks.assert_close(y12, y1 + 2 * y2, "linearity of %d -> %d at 1 M sites" % (cin, cout))


def _strided_sets(loc_in, in_size, size, stride, out_size):
    """(tap, in-site, out-site) triples of a strided rulebook from the closed form of
    SCN/Metadata/RectangularRegions.h:95-119 (output j holds input p iff j*stride <= p <
    j*stride + size, tap = p - j*stride row-major), as three int64 arrays, plus the sorted
    distinct output sites."""
    c = loc_in[:, :3].astype(np.int64)
    taps, ins, outs = [], [], []
    lin_in = _lin(loc_in, in_size)
    for ox in range(size):
        for oy in range(size):
            for oz in range(size):
                o = np.array([ox, oy, oz])
                j = c - o
                ok = ((j % stride == 0) & (j >= 0) & (j // stride < out_size)).all(1)
                jj = j[ok] // stride
                taps.append(np.full(ok.sum(), (ox * size + oy) * size + oz, np.int64))
                ins.append(lin_in[ok])
                outs.append(_lin(np.concatenate([jj, loc_in[ok, 3:]], 1), out_size))
    taps, ins, outs = np.concatenate(taps), np.concatenate(ins), np.concatenate(outs)
    return taps, ins, outs, np.unique(outs)


def _canon(rules, loc_in, in_size, loc_out, out_size):
    li, lo = _lin(loc_in, in_size), _lin(loc_out, out_size)
    t = np.concatenate([np.full(len(r), k, np.int64) for k, r in enumerate(rules)])
    a = np.concatenate([li[r[:, 0]] for r in rules])
    b = np.concatenate([lo[r[:, 1]] for r in rules])
    order = np.lexsort((b, a, t))
    return t[order], a[order], b[order]


@pytest.mark.parametrize("n,spatial", [(60000, 2047), (60000, 255), (3000, 2047), (11200, 601), (12200, 601)])
def test_rulebook_3s2_of_scattered_and_of_dense_points(n, spatial):
    """A 3^3 / stride-2 rulebook of points scattered over a large grid (nearly every output site in a
    64-key block of its own: more blocks than the builder that finds the output sites block by
    block takes, so the candidate sort builds it), of the same number packed into a small grid
    (few, full blocks), of a small scattered set, and of two sets whose output sites fill just under
    and just over the 16 384 blocks that builder takes: both levels' sites and both tables bit-exact
    against numpy, the fine-side table through the transposed rulebook's pooling."""
    from hip_path import HipPath
    g = HipPath(3)
    rng = np.random.default_rng(n + spatial)
    coords = np.unique(np.concatenate([rng.integers(0, spatial, (n, 3)), rng.integers(0, 2, (n, 1))], 1), axis=0)
    coords = coords[rng.permutation(len(coords))].astype(np.int64)
    assert g.input_layer(spatial, coords, 0, 4) == len(coords)
    loc = g.spatial_locations(spatial)
    out = (spatial - 3) // 2 + 1
    rules = g.strided_rules(spatial, out, 3, 2)
    lo = g.spatial_locations(out)
    t, a, b, sites = _strided_sets(loc, spatial, 3, 2, out)
    assert (np.sort(_lin(lo, out)) == sites).all()
    assert (np.diff(lo[:, -1]) >= 0).all()
    order = np.lexsort((b, a, t))
    got = _canon(rules, loc, spatial, lo, out)
    for u, v in zip(got, (t[order], a[order], b[order])):
        assert u.shape == v.shape and (u == v).all()
    # the fine-side table: unpooling adds, into every fine row, the coarse rows of its rules
    y = rng.integers(-8, 8, (len(lo), 4)).astype(np.float32)  # small integers: sums exact in fp32
    up = g.unpool(out, spatial, 3, 2, y)
    want = np.zeros((len(loc), 4), np.float32)
    for r in rules:
        np.add.at(want, r[:, 0], y[r[:, 1]])
    assert (up == want).all()


def test_strided_tree_at_1m_sites():
    """Configuration 4 at its full size: 1 M sites in 4094^3, Convolution 2^3/2 32 -> 64, then
    MaxPooling(3, 2) and Deconvolution 2^3/2 64 -> 32 + BatchNormReLU from the same coarse level.
    Both strided rulebooks (2^3/2 and the 3^3/2 one that needs the candidate sort) and both
    output levels bit-exact against numpy; features through identity taps and by hand."""
    from hip_path import HipPath
    g = HipPath(3)
    coords = synthetic.room_scene(seed=4000, target=1000000, spatial=4094)
    n = len(coords)
    assert g.input_layer(4094, coords, 0, 0) == n
    r1 = g.strided_rules(4094, 2047, 2, 2)
    l1 = g.spatial_locations(2047)
    t, a, b, sites = _strided_sets(coords, 4094, 2, 2, 2047)
    assert (np.sort(_lin(l1, 2047)) == sites).all()
    order = np.lexsort((b, a, t))
    got = _canon(r1, coords, 4094, l1, 2047)
    for u, v in zip(got, (t[order], a[order], b[order])):
        assert u.shape == v.shape and (u == v).all()
    assert sum(len(r) for r in r1) == n  # size = stride: one rule per fine site

    r2 = g.strided_rules(2047, 1023, 3, 2)
    l2 = g.spatial_locations(1023)
    t, a, b, sites2 = _strided_sets(l1, 2047, 3, 2, 1023)
    assert (np.sort(_lin(l2, 1023)) == sites2).all()
    order = np.lexsort((b, a, t))
    got = _canon(r2, l1, 2047, l2, 1023)
    for u, v in zip(got, (t[order], a[order], b[order])):
        assert u.shape == v.shape and (u == v).all()

    rng = np.random.default_rng(40)
    x = rng.normal(size=(n, 32)).astype(np.float32)
    eye_dn = np.zeros((8, 1, 32, 64), np.float32)
    eye_dn[:, 0] = np.eye(32, 64)
    h, macs = g.conv(4094, 2047, 2, 2, x, eye_dn)
    assert macs == float(n) * 32 * 64
    # identity taps: a coarse row is the sum of its children
    parent = _lin(np.concatenate([coords[:, :3] // 2, coords[:, 3:]], 1), 2047)
    lin1 = _lin(l1, 2047)
    row_of = np.searchsorted(lin1[np.argsort(lin1)], parent)
    row_of = np.argsort(lin1)[row_of]
    want = np.zeros((len(l1), 32), np.float64)
    np.add.at(want, row_of, x.astype(np.float64))
    checks.assert_close(h[:, :32], want, "strided convolution with identity taps")
    assert (h[:, 32:] == 0).all()
    # max pooling of ones is one wherever a window holds a site, and the windows' maxima by hand
    mp = g.maxpool(2047, 1023, 3, 2, np.ones((len(l1), 8), np.float32))
    assert mp.shape == (len(l2), 8) and (mp == 1).all()
    hp = rng.normal(size=(len(l1), 64)).astype(np.float32)
    mp = g.maxpool(2047, 1023, 3, 2, hp)
    want = np.zeros((len(l2), 64), np.float32)  # MaxPooling.cpp:50: starts from zero
    for r in r2:
        np.maximum.at(want, r[:, 1], hp[r[:, 0]])
    assert (mp == want).all()
    # transposed convolution with identity taps copies the parent's row; then the batch norm
    eye_up = np.zeros((8, 1, 64, 32), np.float32)
    eye_up[:, 0] = np.eye(64, 32)
    bn = dict(mean=rng.normal(size=32).astype(np.float32), var=rng.uniform(0.5, 1.5, 32).astype(np.float32),
              weight=rng.uniform(0.5, 1.5, 32).astype(np.float32), bias=rng.normal(size=32).astype(np.float32),
              eps=1e-4, leakiness=0.0)
    u, macs = g.deconv(2047, 4094, 2, 2, hp, eye_up)
    assert macs == float(n) * 64 * 32
    assert (u == hp[row_of][:, :32]).all()
    y = g.bn_eval(u, bn["mean"], bn["var"], bn["weight"], bn["bias"], 1e-4, 0.0)
    wgt = bn["weight"] / np.sqrt(bn["var"] + np.float32(1e-4))
    want = np.maximum(u * wgt + (bn["bias"] - bn["mean"] * wgt), 0)
    checks.assert_close(y, want, "batch norm + ReLU behind the transposed convolution")
    fused, _ = g.deconv(2047, 4094, 2, 2, hp, eye_up, None, post=bn)
    checks.assert_close(fused, want, "the same, fused")
    # random weights: three rows by hand through the numpy rule set
    w1 = (rng.normal(size=(8, 1, 32, 64)) * 0.1).astype(np.float32)
    h, _ = g.conv(4094, 2047, 2, 2, x, w1)
    tap = ((coords[:, 0] % 2) * 2 + coords[:, 1] % 2) * 2 + coords[:, 2] % 2
    for row in (0, len(l1) // 2, len(l1) - 1):
        kids = np.nonzero(row_of == row)[0]
        acc = sum(x[i].astype(np.float64) @ w1[tap[i], 0].astype(np.float64) for i in kids)
        checks.assert_close(h[row], acc, "coarse row %d by hand" % row)


def _unet(m=32):
    import torch
    import sparseconvnet_amd as scn
    torch.manual_seed(5)
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 2, [m, 2 * m, 3 * m, 4 * m, 5 * m, 6 * m, 7 * m], False)).add(scn.BatchNormReLU(m)).add(
        scn.OutputLayer(3)).cuda().eval()
    g = torch.Generator().manual_seed(5)
    for mod in model.modules():
        if hasattr(mod, "running_mean"):
            mod.running_mean.copy_(torch.randn(mod.running_mean.shape, generator=g) * 0.1)
            mod.running_var.copy_(torch.rand(mod.running_var.shape, generator=g) + 0.5)
    return model


def test_unet_batch_of_four_scenes_and_1p5m_voxels():
    """Configuration 5's two remaining shapes: a batch of four 1 M-voxel room scenes (the bench batch) and one scene of
    1.5 M voxels (m = 32, 7 levels, mode-4 input with duplicated points).  A cold pass and a pass
    over cached rulebooks are bit-identical; every sample of the batch gets what it gets when it
    runs alone (samples never interact: SCN/Metadata/SubmanifoldConvolutionRules.h:69-81); the
    order of the input points does not matter."""
    import torch
    import sparseconvnet_amd as scn
    model = _unet()
    layer = scn.InputLayer(3, 4096, mode=4)
    rng = np.random.default_rng(50)

    def run(c, f, twice=False):
        with torch.no_grad():
            x = layer([torch.as_tensor(c), torch.as_tensor(f).cuda()])
            y = model(x)
            if twice:
                return y.cpu().numpy(), model(x).cpu().numpy()
            return y.cpu().numpy()

    coords = synthetic.scene_batch(seed=7000, batch=4, target=1000000, spatial=4096, duplicate_fraction=0.3)
    feats = rng.uniform(-1, 1, size=(len(coords), 3)).astype(np.float32)
    cold, warm = run(coords, feats, twice=True)
    assert cold.shape == (len(coords), 32) and np.isfinite(cold).all() and np.abs(cold).max() > 0
    assert (cold == warm).all()
    for b in range(4):
        sel = coords[:, 3] == b
        c1 = coords[sel].copy()
        c1[:, 3] = 0
        alone = run(c1, feats[sel])
        checks.assert_close(cold[sel], alone, "sample %d of the batch against the same scene alone" % b)
    del cold, warm

    coords = synthetic.room_scene(seed=5200, target=1500000, spatial=4096, duplicate_fraction=0.3)
    feats = rng.uniform(-1, 1, size=(len(coords), 3)).astype(np.float32)
    cold, warm = run(coords, feats, twice=True)
    assert cold.shape == (len(coords), 32) and np.isfinite(cold).all() and np.abs(cold).max() > 0
    assert (cold == warm).all()
    perm = rng.permutation(len(coords))
    shuffled = run(coords[perm], feats[perm])
    checks.assert_close(shuffled, cold[perm], "permuted input points at 1.5 M voxels")
