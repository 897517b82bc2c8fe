"""Checks of one implementation of the path against independent statements
(tests/bruteforce.py).  `make(dim)` returns an object with the interface of
oracle.cpu_path.CpuPath; the same checks run on the oracle, on the compiled
reference (where present) and, through an adapter over the C-ABI, on the HIP
library.  Floating-point tolerance: 1e-4 relative, 1e-5 absolute (fp32)."""
import numpy as np

import bruteforce as bf
from oracle.cpu_path import canon_rules

RTOL, ATOL = 1e-4, 1e-5


def assert_close(a, b, what=""):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    assert a.shape == b.shape, (what, a.shape, b.shape)
    if a.size == 0:
        return
    scale = max(1.0, float(np.abs(b).max()))
    err = np.abs(a - b)
    bad = err > ATOL * scale + RTOL * np.abs(b)
    assert not bad.any(), "%s: %d/%d off, max err %g" % (what, bad.sum(), bad.size, err.max())


def check_input_layer(make, dim, mode, seed, n=300, spatial=9, batch=3, with_batch_col=True):
    rng = np.random.default_rng(seed)
    coords = bf.random_sites(rng, dim, spatial, n, batch, duplicates=0 if mode == 0 else n // 2)
    if mode == 0:
        coords = np.unique(coords, axis=0)
        coords = coords[rng.permutation(len(coords))]
    if not with_batch_col:
        coords = coords[coords[:, -1] == 0][:, :dim]
    feats = rng.normal(size=(len(coords), 5)).astype(np.float32)
    p = make(dim)
    n_active = p.input_layer(spatial, coords, 0, mode)
    full = coords if with_batch_col else np.concatenate(
        [coords, np.zeros((len(coords), 1), np.int64)], 1)
    row_of, n_expected = bf.first_occurrence_rows(full)
    if mode == 0:
        assert n_active == len(coords)
        loc = p.spatial_locations(spatial)
        assert (loc == full).all()
        assert_close(p.input_fwd(feats), feats)
        assert_close(p.output_fwd(feats), feats)
        return
    assert n_active == n_expected
    # row numbering: first-occurrence order over the whole input
    loc = p.spatial_locations(spatial)
    assert (loc[row_of] == full).all()
    expect, _ = bf.input_layer_values(full, feats, mode)
    assert_close(p.input_fwd(feats), expect, "input layer mode %d" % mode)
    # rule table: header and per-row lists in input order
    hdr, rows = p.input_rules()
    counts = np.bincount(row_of, minlength=n_expected)
    assert hdr[0] == mode and hdr[2] == len(coords) and hdr[3] == n_expected
    if mode in (3, 4):
        assert hdr[1] == counts.max()
        assert (rows[:, 0] == counts).all()
        for r in range(n_expected):
            assert list(rows[r, 1:1 + counts[r]]) == list(np.nonzero(row_of == r)[0])
    else:
        assert hdr[1] == 1 and (rows[:, 0] == 1).all()
        pick = [np.nonzero(row_of == r)[0][0 if mode == 1 else -1] for r in range(n_expected)]
        assert list(rows[:, 1]) == pick
    # output layer: every input point receives its site's row
    y = rng.normal(size=(n_expected, 4)).astype(np.float32)
    out = p.output_fwd(y)
    if mode in (3, 4):
        assert_close(out, y[row_of], "output layer")
    else:
        picked = np.zeros(len(coords), bool)
        picked[rows[:, 1]] = True
        assert_close(out[picked], y[row_of][picked])
        assert (out[~picked] == 0).all()


def check_mode0_repeated_points(make, dim, seed, n=300, spatial=9, batch=2, cin=3, cout=4):
    """InputLayer mode 0 with a quarter of the points repeated (Metadata/IOLayersRules.h:28-58:
    `mp[p] = i` for every point in turn, so the last point of a site wins).  Every point keeps a
    row of its own (nActive = n, rows in input order, features copied), but only the winner of a
    site is in the grid: the rules of a 3^d convolution connect winners only, and the rows of
    shadowed points receive the bias alone.
    getSpatialLocations: the reference walks the grids (Metadata.cpp:149-170) and leaves the rows
    of shadowed points at zero; the HIP library keeps every point's coordinates.  Both are
    accepted for those rows, the winners' rows must hold their coordinates."""
    rng = np.random.default_rng(seed)
    coords = bf.random_sites(rng, dim, spatial, n, batch, duplicates=n // 4)
    feats = rng.normal(size=(len(coords), cin)).astype(np.float32)
    p = make(dim)
    assert p.input_layer(spatial, coords, 0, 0) == len(coords)
    x = p.input_fwd(feats)
    assert_close(x, feats)
    last = {}
    for i, c in enumerate(map(tuple, coords.tolist())):
        last[c] = i
    winner = np.zeros(len(coords), bool)
    winner[list(last.values())] = True
    assert 0 < (~winner).sum() < len(coords)
    loc = p.spatial_locations(spatial)
    assert loc.shape == coords.shape and (loc[winner] == coords[winner]).all()
    assert (loc[~winner] == 0).all() or (loc[~winner] == coords[~winner]).all()
    rules = p.submanifold_rules(spatial, 3)
    got = set((k, int(i), int(j)) for k, r in enumerate(rules) for i, j in np.asarray(r).reshape(-1, 2).tolist())
    sites = np.array(sorted(last), np.int64)
    want_rules = set((t[0], last[t[1:2 + dim]], last[t[2 + dim:]]) for t in bf.submanifold_triples(sites, dim, 3))
    assert got == want_rules
    assert sum(len(r) for r in rules) == len(got)
    K = 3 ** dim
    w = (rng.normal(size=(K, 1, cin, cout)) * 0.3).astype(np.float32)
    b = rng.normal(size=cout).astype(np.float32)
    y, macs = p.subm_conv(spatial, 3, x, w, b)
    assert macs == len(got) * cin * cout
    want = np.tile(b.astype(np.float64), (len(coords), 1))
    for k, i, j in want_rules:
        want[j] += feats[i].astype(np.float64) @ w[k, 0].astype(np.float64)
    assert_close(y, want.astype(np.float32), "convolution over a mode-0 level with repeated points")
    assert (y[~winner] == b).all()
    # the output layer hands every point its own row back
    assert_close(p.output_fwd(y), y)
    # a strided rulebook over the same level: its rules start from the winners only
    # (Metadata/ConvolutionRules.h:61-105 walks the input grids)
    if spatial % 2 == 1:
        out3 = (spatial - 3) // 2 + 1
        srules = p.strided_rules(spatial, out3, 3, 2)
        loc_out = p.spatial_locations(out3)
        got_s = set()
        for k, r in enumerate(srules):
            for i, j in np.asarray(r).reshape(-1, 2).tolist():
                got_s.add((k, int(i)) + tuple(loc_out[j].tolist()))
        want_s = set((t[0], last[t[1:2 + dim]]) + t[2 + dim:] for t in bf.strided_triples(sites, dim, 3, 2, out3))
        assert got_s == want_s
        assert sum(len(r) for r in srules) == len(got_s)
    # filter 2 / stride 2 over a size that halves exactly (the builders' path without a sort), and
    # once more from the level that made, which has no repeated keys
    if spatial % 4 == 0:
        half = spatial // 2
        srules = p.strided_rules(spatial, half, 2, 2)
        loc_out = p.spatial_locations(half)
        got_s = set()
        for k, r in enumerate(srules):
            for i, j in np.asarray(r).reshape(-1, 2).tolist():
                got_s.add((k, int(i)) + tuple(loc_out[j].tolist()))
        want_s = set((t[0], last[t[1:2 + dim]]) + t[2 + dim:] for t in bf.strided_triples(sites, dim, 2, 2, half))
        assert got_s == want_s
        assert sum(len(r) for r in srules) == len(got_s)
        assert len(loc_out) == len(set(t[2:] for t in want_s))
        rules2 = p.strided_rules(half, half // 2, 2, 2)
        loc2 = p.spatial_locations(half // 2)
        row_of = {tuple(c): i for i, c in enumerate(loc_out.tolist())}
        got2 = set((k, int(i)) + tuple(loc2[j].tolist()) for k, r in enumerate(rules2)
                   for i, j in np.asarray(r).reshape(-1, 2).tolist())
        want2 = set((t[0], row_of[t[1:2 + dim]]) + t[2 + dim:]
                    for t in bf.strided_triples(np.array(sorted(row_of), np.int64), dim, 2, 2, half // 2))
        assert got2 == want2


def check_bl_input_layer(make, dim, mode, seed, batch=3, length=70, spatial=9, planes=5, empties=True):
    """BLInputLayer / BLOutputLayer against a per-sample dictionary: row numbering, rule table,
    merged features (mode 1 = last point of a site, 2 = first, 3 = sum, 4 = mean) and the way
    back, with zeros at empty positions."""
    rng = np.random.default_rng(seed)
    coords = rng.integers(0, spatial, (batch, length, dim)).astype(np.int64)
    if mode == 0:  # unique inside a sample, nothing empty
        for b in range(batch):
            cells = rng.permutation(spatial ** dim)[:length]
            coords[b] = np.stack(np.unravel_index(cells, (spatial,) * dim), 1)
    elif empties:
        hole = rng.random((batch, length)) < 0.2
        coords[hole] = -1
        if batch > 2:
            coords[1, :, :] = -1  # a sample without points still counts
    feats = rng.normal(size=(batch, length, planes)).astype(np.float32)
    flat = feats.reshape(-1, planes)
    p = make(dim)
    n_active = p.bl_input_layer(spatial, coords, mode)
    hdr, rows = p.bl_rules()
    if mode == 0:
        assert n_active == batch * length and list(hdr) == [0, 1, batch, length, batch * length]
        loc = p.spatial_locations(spatial)
        want = np.concatenate([coords.reshape(-1, dim), np.repeat(np.arange(batch), length)[:, None]], 1)
        assert (loc == want).all()
        assert_close(p.bl_input_fwd(feats), flat)
        assert_close(p.bl_output_fwd(flat), feats)
        assert p.batch_size(spatial) == batch
        return
    groups, loc_want = bf.bl_groups(coords)
    assert n_active == len(groups) and p.nactive(spatial) == len(groups)
    assert (p.spatial_locations(spatial) == loc_want).all()
    assert p.batch_size(spatial) == batch
    longest = max([len(g) for g in groups] + [1])
    assert list(hdr) == [mode, longest if mode >= 3 else 1, batch, length, len(groups)]
    expect = np.zeros((len(groups), planes), np.float64)
    for r, g in enumerate(groups):
        if mode == 1:
            assert list(rows[r]) == [1, g[-1]]
            expect[r] = flat[g[-1]]
        elif mode == 2:
            assert list(rows[r]) == [1, g[0]]
            expect[r] = flat[g[0]]
        else:
            assert rows[r, 0] == len(g) and list(rows[r, 1:1 + len(g)]) == g and (rows[r, 1 + len(g):] == 0).all()
            expect[r] = flat[g].astype(np.float64).sum(0) / (len(g) if mode == 4 else 1)
    assert_close(p.bl_input_fwd(feats), expect, "batch-by-length input, mode %d" % mode)
    y = rng.normal(size=(len(groups), 4)).astype(np.float32)
    back = np.zeros((batch * length, 4), np.float32)
    for r, g in enumerate(groups):
        listed = g if mode >= 3 else [g[-1] if mode == 1 else g[0]]
        back[listed] = y[r]
    out = p.bl_output_fwd(y)
    assert out.shape == (batch, length, 4)
    assert_close(out.reshape(-1, 4), back, "batch-by-length output, mode %d" % mode)


def check_input_batch(make, dim, seed, spatial=9, planes=4):
    """The point-at-a-time route (sparseconvnet/inputBatch.py) against a dictionary: calls with
    and without a sample column, repeated sites inside and across calls with and without
    overwrite, single points, samples that stay empty, a batch that grows through the sample
    column, and a sample taken from a dense block that hangs over the edge of the grid."""
    rng = np.random.default_rng(seed)
    p = make(dim)
    p.batch_begin(spatial)
    table = bf.PointTable()

    def put(locations, overwrite, sample=None):
        vectors = rng.normal(size=(len(locations), planes)).astype(np.float32)
        p.batch_set_locations(locations, vectors, overwrite)
        for l, v in zip(locations, vectors):
            table.set(tuple(l) if sample is None else tuple(l) + (sample,), v, overwrite)

    def sites(n):  # repeats are likely: 9^dim cells at most
        return rng.integers(0, spatial, size=(n, dim)).astype(np.int64)

    p.batch_add_sample()                       # sample 0
    a = sites(60)
    put(a, False, 0)
    put(np.concatenate([a[:20], sites(15)]), True, 0)
    put(a[10:30], False, 0)                    # known sites, no overwrite: nothing changes
    p.batch_add_sample()                       # sample 1 stays empty
    p.batch_add_sample()                       # sample 2
    put(sites(40), False, 2)
    for _ in range(5):
        put(sites(1), bool(rng.integers(0, 2)), 2)
    # (the reference's pointer to the current sample does not survive a batch that grows through
    # the sample column or a dense block: after those, only calls that name the sample, until
    # the next add_sample)
    with_sample = np.concatenate([sites(50), rng.choice([0, 2, 4], size=(50, 1))], 1).astype(np.int64)
    put(with_sample, False)                    # the batch grows to 5 samples
    again = np.concatenate([with_sample[:25], with_sample[:10], with_sample[40:]])
    put(again, True)                           # repeats inside one overwriting call: the last one stays
    p.batch_add_sample()                       # sample 5
    put(sites(30), True, 5)
    block = rng.normal(size=(4,) * dim + (planes,)).astype(np.float32)
    block[np.abs(block).max(-1) < 0.9] *= 0.1  # some cells below the threshold
    offset = np.array([spatial - 2] + [-1] * (dim - 1), np.int64)
    p.batch_add_sample_from_tensor(block, offset, 0.5)   # sample 6
    table.dense_block(block, offset, spatial, 6, 0.5)
    put(np.concatenate([sites(10), np.full((10, 1), 6)], 1).astype(np.int64), True)
    p.batch_end()

    assert p.nactive(spatial) == len(table.rows)
    assert p.batch_size(spatial) == 7
    assert (p.spatial_locations(spatial) == table.locations()).all()   # rows: order of first appearance
    feats = p.batch_features()
    assert feats.shape == (len(table.rows), planes) and (feats == table.features()).all()
    # the level is an ordinary one: its rulebooks come out as for any other input route
    loc = p.spatial_locations(spatial)
    rules = p.submanifold_rules(spatial, 3)
    assert bf.triples_of(canon_rules(rules, loc, loc)) == bf.submanifold_triples(loc, dim, 3)


def check_generate_rulebooks(make, dim, size, spatial, seed, n=400, batch=2):
    """Rulebooks built ahead of their use (InputBatch.precompute_metadata): every level down to
    the first whose extent does not halve exists afterwards, none beyond it, and the
    rulebooks are the ones an explicit request gives."""
    rng = np.random.default_rng(seed)
    spatial = np.broadcast_to(np.asarray(spatial, np.int64), (dim,))
    coords = np.concatenate([np.stack([rng.integers(0, s, n) for s in spatial], 1),
                             rng.integers(0, batch, size=(n, 1))], 1).astype(np.int64)
    p, q = make(dim), make(dim)
    p.input_layer(spatial, coords, 0, 3)
    q.input_layer(spatial, coords, 0, 3)
    p.generate_rulebooks(size)
    levels = [spatial]
    while all(s >= size and s % 2 == (size == 3) for s in levels[-1]):
        levels.append(levels[-1] // 2 if size == 2 else (levels[-1] - 1) // 2)
    assert len(levels) >= 3
    for fine, coarse in zip(levels, levels[1:]):
        assert p.nactive(coarse) > 0                       # built by generate_rulebooks alone
        r_q = q.strided_rules(fine, coarse, size, 2)
        assert p.nactive(coarse) == q.nactive(coarse)
        lf, lc = p.spatial_locations(fine), p.spatial_locations(coarse)
        r_p = p.strided_rules(fine, coarse, size, 2)
        assert bf.triples_of(canon_rules(r_p, lf, lc)) == bf.strided_triples(lf, dim, size, 2, coarse)
        assert bf.triples_of(canon_rules(r_p, lf, lc)) == bf.triples_of(
            canon_rules(r_q, q.spatial_locations(fine), q.spatial_locations(coarse)))
    for lvl in levels:
        loc = p.spatial_locations(lvl)
        assert bf.triples_of(canon_rules(p.submanifold_rules(lvl, 3), loc, loc)) == bf.submanifold_triples(loc, dim, 3)
    beyond = levels[-1] // 2 if size == 2 else np.maximum((levels[-1] - 1) // 2, 0)
    if not any((beyond == l).all() for l in levels):
        assert p.nactive(beyond) == 0


def _setup(make, dim, spatial, n, batch, seed, C):
    rng = np.random.default_rng(seed)
    coords = bf.random_sites(rng, dim, spatial, n, batch, duplicates=n // 4)
    feats = rng.normal(size=(len(coords), C)).astype(np.float32)
    p = make(dim)
    p.input_layer(spatial, coords, 0, 3)
    loc = p.spatial_locations(spatial)
    x = p.input_fwd(feats)
    return rng, p, loc, x


def check_submanifold(make, dim, size, seed, spatial=8, n=200, batch=2, cin=3, cout=4, bias=False):
    rng, p, loc, x = _setup(make, dim, spatial, n, batch, seed, cin)
    rules = p.submanifold_rules(spatial, size)
    K = int(np.prod(np.broadcast_to(np.asarray(size), (dim,))))
    assert len(rules) == K
    got = bf.triples_of(canon_rules(rules, loc, loc))
    assert got == bf.submanifold_triples(loc, dim, size)
    assert sum(len(r) for r in rules) == len(got)  # no duplicate rules
    for r in rules:  # at most one rule per (offset, output row)
        assert len(np.unique(r[:, 1])) == len(r)
    sz = np.broadcast_to(np.asarray(size), (dim,))
    if (sz % 2 == 1).all():
        centre = rules[K // 2]  # centre tap = identity on all rows
        assert len(centre) == len(loc) and (centre[:, 0] == centre[:, 1]).all()
        # symmetry (k, i, j) <-> (K-1-k, j, i)
        for k in range(K):
            a = set(map(tuple, rules[k].tolist()))
            b = set((j, i) for i, j in rules[K - 1 - k].tolist())
            assert a == b
    w = (rng.normal(size=(K, 1, cin, cout)) * 0.3).astype(np.float32)
    b = rng.normal(size=cout).astype(np.float32) if bias else None
    y, macs = p.subm_conv(spatial, size, x, w, b)
    assert macs == len(got) * cin * cout
    assert_close(y, bf.dense_subm_conv(loc, x, w, spatial, size, batch, b), "submanifold conv")


def check_strided(make, dim, size, stride, seed, out_spatial=4, n=150, batch=2, cin=3, cout=4,
                  bias=False):
    size_a = np.broadcast_to(np.asarray(size), (dim,))
    stride_a = np.broadcast_to(np.asarray(stride), (dim,))
    out_sp = np.broadcast_to(np.asarray(out_spatial), (dim,))
    in_sp = (out_sp - 1) * stride_a + size_a
    rng = np.random.default_rng(seed)
    pts = np.stack([rng.integers(0, s, n) for s in in_sp], 1)
    coords = np.concatenate([pts, rng.integers(0, batch, (n, 1))], 1).astype(np.int64)
    feats = rng.normal(size=(n, cin)).astype(np.float32)
    p = make(dim)
    p.input_layer(in_sp, coords, 0, 4)
    loc = p.spatial_locations(in_sp)
    x = p.input_fwd(feats)
    rules = p.strided_rules(in_sp, out_sp, size, stride)
    K = int(size_a.prod())
    assert len(rules) == K
    loc_out = p.spatial_locations(out_sp)
    assert p.nactive(out_sp) == len(loc_out)
    expect = bf.strided_triples(loc, dim, size, stride, out_sp)
    got = bf.triples_of(canon_rules(rules, loc, loc_out))
    assert got == expect
    assert sum(len(r) for r in rules) == len(expect)
    # active outputs = exactly the sites with at least one rule, each listed once
    want_out = set(t[1 + dim + 1:] for t in expect)
    assert set(map(tuple, loc_out.tolist())) == want_out and len(loc_out) == len(want_out)
    for r in rules:
        assert len(np.unique(r[:, 1])) == len(r)
    assert p.batch_size(out_sp) == p.batch_size(in_sp)
    # rows of one sample are contiguous and samples ascend at a created level
    assert (np.diff(loc_out[:, -1]) >= 0).all()

    w = (rng.normal(size=(K, 1, cin, cout)) * 0.3).astype(np.float32)
    b = rng.normal(size=cout).astype(np.float32) if bias else None
    y, macs = p.conv(in_sp, out_sp, size, stride, x, w, b)
    assert macs == len(expect) * cin * cout
    dense_ok = dim <= 3   # torch has dense convolutions and pooling up to three dimensions
    rows = None if dense_ok else bf.rule_rows(expect, loc, loc_out)
    want = {}
    if dense_ok:
        want["conv"] = bf.sample_dense(bf.dense_strided_conv(loc, x, w, in_sp, size, stride, batch, b), loc_out)
    else:
        want["conv"] = bf.rows_strided_ops(rows, x, np.zeros((len(loc_out), 1), np.float32), w,
                                           np.zeros((K, 1, 1, 1), np.float32), len(loc), len(loc_out), K, b)[0]
    assert_close(y, want["conv"], "strided conv")
    if not dense_ok:
        w2 = (rng.normal(size=(K, 1, cout, cin)) * 0.3).astype(np.float32)
        _, want_mp, want_ap, want_up, want_dz = bf.rows_strided_ops(rows, x, y, w, w2, len(loc), len(loc_out), K)
        assert_close(p.maxpool(in_sp, out_sp, size, stride, x), want_mp, "max pooling")
        assert_close(p.avgpool(in_sp, out_sp, size, stride, x), want_ap, "average pooling")
        assert_close(p.unpool(out_sp, in_sp, size, stride, y), want_up, "unpooling")
        z, macs2 = p.deconv(out_sp, in_sp, size, stride, y, w2)
        assert macs2 == len(expect) * cin * cout
        assert_close(z, want_dz, "deconvolution")
        return p
    # max pooling over the same rulebook: zero-initialised, so max(0, active inputs)
    mp = p.maxpool(in_sp, out_sp, size, stride, x)
    dmp = bf.dense_maxpool(loc, x, in_sp, size, stride, batch)
    assert_close(mp, bf.sample_dense(dmp, loc_out), "max pooling")
    mp1 = p.maxpool(in_sp, out_sp, size, stride, x, 1)
    assert_close(mp1, mp[:, 1:], "max pooling nFeaturesToDrop")
    # average pooling: window sum over the filter volume, absent sites count as zeros
    ap = p.avgpool(in_sp, out_sp, size, stride, x)
    dap = bf.dense_avgpool(loc, x, in_sp, size, stride, batch)
    assert_close(ap, bf.sample_dense(dap, loc_out), "average pooling")
    assert_close(p.avgpool(in_sp, out_sp, size, stride, x, 2), ap[:, 2:], "average pooling nFeaturesToDrop")
    # unpooling: the transposed convolution whose every tap is the identity matrix
    eye = np.broadcast_to(np.eye(cout, dtype=np.float32), (K, 1, cout, cout)).copy()
    up = p.unpool(out_sp, in_sp, size, stride, y)
    dup = bf.dense_deconv(loc_out, y, eye, out_sp, size, stride, batch)
    assert_close(up, bf.sample_dense(dup, loc), "unpooling")
    assert_close(p.unpool(out_sp, in_sp, size, stride, y, 1), up[:, 1:], "unpooling nFeaturesToDrop")
    # deconvolution back to the fine level: transposed conv masked to the fine active set
    w2 = (rng.normal(size=(K, 1, cout, cin)) * 0.3).astype(np.float32)
    z, macs2 = p.deconv(out_sp, in_sp, size, stride, y, w2)
    assert macs2 == len(expect) * cin * cout
    dz = bf.dense_deconv(loc_out, y, w2, out_sp, size, stride, batch)
    assert_close(z, bf.sample_dense(dz, loc), "deconvolution")
    return p


def check_bn(make, seed, n=257, C=13):
    rng = np.random.default_rng(seed)
    import torch
    import torch.nn.functional as F
    x = rng.normal(size=(n, C)).astype(np.float32)
    mean = rng.normal(size=C).astype(np.float32)
    var = rng.uniform(0.5, 1.5, C).astype(np.float32)
    g = rng.normal(size=C).astype(np.float32)
    b = rng.normal(size=C).astype(np.float32)
    p = make(2)
    for leak in (0.0, 0.333, 1.0):
        for affine in (True, False):
            y = p.bn_eval(x, mean, var, g if affine else None, b if affine else None, 1e-4, leak)
            t = F.batch_norm(torch.as_tensor(x, dtype=torch.float64), torch.as_tensor(mean).double(),
                             torch.as_tensor(var).double(),
                             torch.as_tensor(g).double() if affine else None,
                             torch.as_tensor(b).double() if affine else None, False, 0.0, 1e-4)
            t = torch.where(t > 0, t, t * leak)
            assert_close(y, t.numpy(), "bn leak=%g" % leak)


def check_nin(make, seed, shapes=((257, 13, 7), (64, 32, 32), (1, 5, 3), (300, 64, 96), (0, 4, 4))):
    """NetworkInNetwork against the float64 matrix product of numpy, with and without bias."""
    rng = np.random.default_rng(seed)
    p = make(3)
    for n, cin, cout in shapes:
        x = rng.normal(size=(n, cin)).astype(np.float32)
        w = (rng.normal(size=(cin, cout)) * 0.3).astype(np.float32)
        b = rng.normal(size=cout).astype(np.float32)
        for bias in (None, b):
            y, macs = p.nin(x, w, bias)
            expect = x.astype(np.float64) @ w.astype(np.float64) + (0 if bias is None else bias.astype(np.float64))
            assert y.shape == (n, cout)
            assert_close(y, expect, "network in network %s" % ((n, cin, cout),))
            assert macs == n * cin * cout


def check_s2d(make, dim, seed, spatial=6, n=80, batch=3, C=4):
    rng, p, loc, x = _setup(make, dim, spatial, n, batch, seed, C)
    d = p.s2d(spatial, x)
    assert d.shape == (batch, C) + (spatial,) * dim
    assert_close(d, bf.to_dense(loc, x, spatial, batch).numpy(), "sparse to dense")
    rules = p.s2d_rules(spatial)
    assert len(rules) == batch
    for b, r in enumerate(rules):
        sel = loc[r[:, 0]]
        assert (sel[:, -1] == b).all()
        off = np.ravel_multi_index(tuple(sel[:, i] for i in range(dim)), (spatial,) * dim)
        assert (off == r[:, 1]).all()
    assert sum(len(r) for r in rules) == len(loc)


def check_active_pooling(make, dim, seed, spatial=6, n=90, batch=4, C=5):
    """ActivePooling forward and backward (CPU/ActivePooling.cpp:8-83) against the closed form: per
    sample the sum / mean of its rows, and that sample's gradient (times 1 / count) back to each of
    its rows.  Two inputs: samples of many sites, one of them empty (where the compiled reference's
    rule builder does not return and its adapter answers None), and samples of exactly one site
    each (where it returns: the one input on which the reference itself can be asked)."""
    rng = np.random.default_rng(seed)
    for single in (False, True):
        if single:
            coords = np.concatenate([rng.integers(0, spatial, size=(batch, dim)), np.arange(batch)[:, None]], 1)
        else:
            coords = bf.random_sites(rng, dim, spatial, n, batch, duplicates=n // 4)
            coords = coords[coords[:, -1] != 1]  # sample 1 stays empty
        feats = rng.normal(size=(len(coords), C)).astype(np.float32)
        p = make(dim)
        p.input_layer(spatial, coords, batch, 3)
        loc = p.spatial_locations(spatial)
        x = p.input_fwd(feats)
        d_out = rng.normal(size=(batch, C)).astype(np.float32)
        for average in (False, True):
            got = p.active_pooling(spatial, x, average)
            got_b = p.active_pooling_bwd(spatial, d_out, average)
            if got is None:  # the compiled reference on an input its rule builder cannot handle
                assert not single and got_b is None
                continue
            want = np.zeros((batch, C))
            count = np.bincount(loc[:, -1], minlength=batch)
            np.add.at(want, loc[:, -1], x.astype(np.float64))
            mult = np.where(count > 0, 1.0 / np.maximum(count, 1), 1.0) if average else np.ones(batch)
            assert got.shape == (batch, C)
            assert_close(got, want * mult[:, None], "active pooling, average=%s" % average)
            assert_close(got_b, (d_out * mult[:, None])[loc[:, -1]], "active pooling gradient, average=%s" % average)
        if single:
            assert got is not None


def check_level_replacement(make, seed=11):
    """What happens to a level that is built twice, as the reference does it
    (Metadata/ConvolutionRules.h:68-70, Metadata/Metadata.cpp:492-518, CPU/Deconvolution.cpp:15-18):
    operations with the same (input size, filter, stride) share one rulebook and one output
    level; a strided rulebook with another key that lands on an existing spatial size builds
    that level anew from its own input; a deconvolution towards a spatial size that was never
    built finds an empty fine level, yields no rows and leaves the coarse level empty."""
    rng = np.random.default_rng(seed)
    dim, batch = 2, 2
    coords = bf.random_sites(rng, dim, 9, 60, batch)
    coords = np.unique(coords, axis=0)
    x = rng.normal(size=(len(coords), 3)).astype(np.float32)
    p = make(dim)
    p.input_layer(9, coords, 0, 0)
    loc = p.spatial_locations(9)
    w = (rng.normal(size=(9, 1, 3, 2)) * 0.3).astype(np.float32)
    y, _ = p.conv(9, 4, 3, 2, x, w)
    loc_a = p.spatial_locations(4)
    want_a = set(t[1 + dim + 1:] for t in bf.strided_triples(loc, dim, 3, 2, np.array([4, 4])))
    assert set(map(tuple, loc_a.tolist())) == want_a
    mp = p.maxpool(9, 4, 3, 2, x)  # same key: same rulebook, level untouched
    assert (p.spatial_locations(4) == loc_a).all() and mp.shape == (len(loc_a), 3)
    # another key onto spatial size 4: the level is rebuilt from this rulebook's outputs
    w6 = (rng.normal(size=(36, 1, 3, 2)) * 0.1).astype(np.float32)
    y6, _ = p.conv(9, 4, 6, 1, x, w6)
    loc_b = p.spatial_locations(4)
    want_b = set(t[1 + dim + 1:] for t in bf.strided_triples(loc, dim, 6, 1, np.array([4, 4])))
    assert set(map(tuple, loc_b.tolist())) == want_b and p.nactive(4) == len(want_b) == len(y6)
    dense = bf.dense_strided_conv(loc, x, w6, 9, 6, 1, batch)
    assert_close(y6, bf.sample_dense(dense, loc_b), "second rulebook onto the same level")
    # deconvolution towards a level nobody built: 4 -> (4-1)*3+3 = 12
    wd = (rng.normal(size=(9, 1, 2, 3)) * 0.3).astype(np.float32)
    z, macs = p.deconv(4, 12, 3, 3, y6, wd)
    assert z.shape == (0, 3) and macs == 0
    assert p.nactive(12) == 0 and p.nactive(4) == 0


def check_special_values(make, seed=12):
    """NaN, infinities, negative zero and all-negative windows: max pooling starts from zero and
    replaces only when `out < in` (CPU/MaxPooling.cpp:17-18,50), so a NaN never enters and an
    all-negative window gives +0; batch norm multiplies by the leakiness where y > 0 is false
    (CPU/BatchNormalization.cpp:55-58), so ReLU maps negatives to -0.0 and NaN stays NaN."""
    rng = np.random.default_rng(seed)
    dim, batch = 2, 1
    coords = np.unique(bf.random_sites(rng, dim, 8, 50, batch), axis=0)
    n = len(coords)
    x = rng.normal(size=(n, 4)).astype(np.float32)
    x[rng.random(n) < 0.2, 0] = np.nan
    x[:, 1] = -np.abs(x[:, 1]) - 0.5            # every window negative
    x[rng.random(n) < 0.3, 2] = -0.0
    x[rng.random(n) < 0.1, 3] = np.inf
    p = make(dim)
    p.input_layer(8, coords, 0, 0)
    loc = p.spatial_locations(8)
    rules = p.strided_rules(8, 4, 2, 2)
    got = p.maxpool(8, 4, 2, 2, x)
    want = np.zeros_like(got)
    for r in rules:
        for i, o in r:
            lt = want[o] < x[i]                 # false for NaN
            want[o][lt] = x[i][lt]
    assert got.shape == want.shape
    assert (np.isnan(got) == np.isnan(want)).all() and not np.isnan(got).any()
    assert (got == want).all() and (np.signbit(got) == np.signbit(want)).all()
    assert (got[:, 1] == 0).all() and not np.signbit(got[:, 1]).any()
    mean, var = np.zeros(4, np.float32), np.ones(4, np.float32)
    y = p.bn_eval(x, mean, var, None, None, 1e-4, 0.0)
    w = np.float32(1.0) / np.sqrt(var + np.float32(1e-4))
    b = -mean * w + np.float32(0)               # the reference's shift term: +0 here
    t = x * w + b
    with np.errstate(invalid="ignore"):
        want = t * np.where(t > 0, np.float32(1), np.float32(0))
    assert (np.isnan(y) == np.isnan(want)).all()
    ok = np.isfinite(want)
    assert (np.isinf(y) == np.isinf(want)).all()
    assert_close(y[ok], want[ok], "batch norm special values")
    ok = ~np.isnan(want)
    assert (np.signbit(y[ok]) == np.signbit(want[ok])).all()   # negatives become -0.0, as in the reference


def check_empty(make, dim=3):
    """Zero active sites: every op returns an empty result and 0 multiply-adds."""
    p = make(dim)
    n = p.input_layer(8, np.zeros((0, dim + 1), np.int64), 0, 3)
    assert n == 0
    rules = p.submanifold_rules(8, 3)
    assert sum(len(r) for r in rules) == 0
    y, macs = p.subm_conv(8, 3, np.zeros((0, 3), np.float32), np.ones((27, 1, 3, 2), np.float32))
    assert y.shape == (0, 2) and macs == 0


# ---- backward pass ------------------------------------------------------------------------------
# Independent statement: torch.autograd through the dense equivalents (conv / conv_transpose /
# pooling / batch_norm on a zero-filled dense tensor), in float64; for dimensions torch has no
# dense routines for, loops over the brute-force rule set.

def _t64(a, grad=False):
    import torch
    return torch.tensor(np.asarray(a, np.float64), dtype=torch.float64, requires_grad=grad)


def _dense_t(loc, feats_t, spatial, batch):
    """Differentiable bf.to_dense."""
    import torch
    dim = loc.shape[1] - 1
    spatial = [int(s) for s in np.broadcast_to(np.asarray(spatial), (dim,))]
    d = torch.zeros([batch, feats_t.shape[1]] + spatial, dtype=torch.float64)
    return _index_put(d, loc, feats_t)


def _index_put(d, loc, feats_t):
    import torch
    dim = loc.shape[1] - 1
    d = d.movedim(1, -1).clone()  # [B, spatial..., C]
    idx = (torch.as_tensor(loc[:, -1]),) + tuple(torch.as_tensor(loc[:, i]) for i in range(dim))
    d = d.index_put(idx, feats_t)
    return d.movedim(-1, 1)


def _sample_t(dense, loc):
    import torch
    dim = loc.shape[1] - 1
    idx = (torch.as_tensor(loc[:, -1]),) + tuple(torch.as_tensor(loc[:, i]) for i in range(dim))
    return dense.movedim(1, -1)[idx]


def _grads(loss, *leaves):
    loss.backward()
    return [None if v is None else v.grad.numpy() for v in leaves]


def _triple_grads(rows, x, d_out, w, n_in_rows):
    """d_in, d_w by loops over (k, in row, out row) rules."""
    d_in = np.zeros((n_in_rows, w.shape[2]))
    d_w = np.zeros(w.shape, np.float64)
    for k, i, j in rows:
        d_in[i] += d_out[j].astype(np.float64) @ w[k, 0].astype(np.float64).T
        d_w[k, 0] += np.outer(x[i].astype(np.float64), d_out[j].astype(np.float64))
    return d_in, d_w


def check_conv_backward(make, dim, size, seed, spatial=8, n=200, batch=2, cin=5, cout=4, bias=True):
    """SubmanifoldConvolution backward (CPU/Convolution.cpp:152-185)."""
    import torch
    rng, p, loc, x = _setup(make, dim, spatial, n, batch, seed, cin)
    K = int(np.prod(np.broadcast_to(np.asarray(size), (dim,))))
    w = (rng.normal(size=(K, 1, cin, cout)) * 0.3).astype(np.float32)
    d_out = rng.normal(size=(len(loc), cout)).astype(np.float32)
    d_in, d_w, d_b = p.subm_conv_bwd(spatial, size, x, d_out, w, with_bias=bias)
    if dim in bf._CONV:
        xt, wt = _t64(x, True), _t64(w, True)
        bt = _t64(np.zeros(cout), True)
        sz = [int(s) for s in np.broadcast_to(np.asarray(size), (dim,))]
        pads = []
        for s in reversed(sz):
            pads += [s // 2, s - 1 - s // 2]
        y = bf._CONV[dim](torch.nn.functional.pad(_dense_t(loc, xt, spatial, batch), pads),
                          bf.dense_weight(wt, dim, sz), bt)
        gx, gw, gb = _grads((_sample_t(y, loc) * _t64(d_out)).sum(), xt, wt, bt)
    else:
        rows = bf.rule_rows(bf.submanifold_triples(loc, dim, size), loc, loc)
        gx, gw = _triple_grads(rows, x, d_out, w, len(loc))
        gb = d_out.astype(np.float64).sum(0)
    assert_close(d_in, gx, "submanifold d_input")
    assert_close(d_w, gw, "submanifold d_weight")
    if bias:
        assert_close(d_b, gb, "submanifold d_bias")
    else:
        assert d_b is None
    return p


def check_strided_backward(make, dim, size, stride, seed, out_spatial=4, n=150, batch=2, cin=5, cout=4, pools=True):
    """Convolution, Deconvolution, MaxPooling, AveragePooling and UnPooling backward over one
    strided rulebook (CPU/Convolution.cpp:81-115, CPU/Deconvolution.cpp:43-77,
    CPU/MaxPooling.cpp:21-35,61-87, CPU/AveragePooling.cpp:21-35,62-86, CPU/UnPooling.cpp:21-32,58-78)."""
    import torch
    F = torch.nn.functional
    size_a = np.broadcast_to(np.asarray(size), (dim,))
    stride_a = np.broadcast_to(np.asarray(stride), (dim,))
    out_sp = np.broadcast_to(np.asarray(out_spatial), (dim,))
    in_sp = (out_sp - 1) * stride_a + size_a
    rng = np.random.default_rng(seed)
    pts = np.stack([rng.integers(0, s, n) for s in in_sp], 1)
    coords = np.concatenate([pts, rng.integers(0, batch, (n, 1))], 1).astype(np.int64)
    p = make(dim)
    p.input_layer(in_sp, coords, 0, 4)
    loc = p.spatial_locations(in_sp)
    x = p.input_fwd(rng.normal(size=(n, cin)).astype(np.float32))
    p.strided_rules(in_sp, out_sp, size, stride)
    loc_out = p.spatial_locations(out_sp)
    K = int(size_a.prod())
    st = [int(s) for s in stride_a]
    sz = [int(s) for s in size_a]
    w = (rng.normal(size=(K, 1, cin, cout)) * 0.3).astype(np.float32)
    d_y = rng.normal(size=(len(loc_out), cout)).astype(np.float32)
    d_in, d_w, d_b = p.conv_bwd(in_sp, out_sp, size, stride, x, d_y, w, with_bias=True)
    xt, wt, bt = _t64(x, True), _t64(w, True), _t64(np.zeros(cout), True)
    y = bf._CONV[dim](_dense_t(loc, xt, in_sp, batch), bf.dense_weight(wt, dim, sz), bt, stride=st)
    gx, gw, gb = _grads((_sample_t(y, loc_out) * _t64(d_y)).sum(), xt, wt, bt)
    assert_close(d_in, gx, "strided d_input")
    assert_close(d_w, gw, "strided d_weight")
    assert_close(d_b, gb, "strided d_bias")
    # transposed convolution: coarse rows in, fine rows out
    yc = rng.normal(size=(len(loc_out), cout)).astype(np.float32)
    w2 = (rng.normal(size=(K, 1, cout, cin)) * 0.3).astype(np.float32)
    d_z = rng.normal(size=(len(loc), cin)).astype(np.float32)
    d_in, d_w, d_b = p.deconv_bwd(out_sp, in_sp, size, stride, yc, d_z, w2, with_bias=True)
    yt, wt, bt = _t64(yc, True), _t64(w2, True), _t64(np.zeros(cin), True)
    wd = bf.dense_weight(wt, dim, sz).transpose(0, 1).contiguous()
    z = bf._CONVT[dim](_dense_t(loc_out, yt, out_sp, batch), wd, bt, stride=st)
    gy, gw, gb = _grads((_sample_t(z, loc) * _t64(d_z)).sum(), yt, wt, bt)
    assert_close(d_in, gy, "transposed d_input")
    assert_close(d_w, gw, "transposed d_weight")
    assert_close(d_b, gb, "transposed d_bias")
    if not pools:  # (the pooling checks below drop two planes: they need more than two)
        return p
    # max pooling (from zero: a window of negative values passes no gradient)
    mp = p.maxpool(in_sp, out_sp, size, stride, x)
    d_mp = rng.normal(size=mp.shape).astype(np.float32)
    got = p.maxpool_bwd(in_sp, out_sp, size, stride, x, mp, d_mp)
    xt = _t64(x, True)
    dense = bf._POOL[dim](_dense_t(loc, xt, in_sp, batch), sz, st).clamp(min=0)
    (gx,) = _grads((_sample_t(dense, loc_out) * _t64(d_mp)).sum(), xt)
    assert_close(got, gx, "max pooling d_input")
    # average pooling
    got = p.avgpool_bwd(in_sp, out_sp, size, stride, cin, d_mp)
    xt = _t64(x, True)
    dense = bf._AVG[dim](_dense_t(loc, xt, in_sp, batch), sz, st)
    (gx,) = _grads((_sample_t(dense, loc_out) * _t64(d_mp)).sum(), xt)
    assert_close(got, gx, "average pooling d_input")
    got2 = p.avgpool_bwd(in_sp, out_sp, size, stride, cin, d_mp[:, 2:], 2)
    assert (got2[:, :2] == 0).all()
    assert_close(got2[:, 2:], gx[:, 2:], "average pooling d_input, nFeaturesToDrop")
    # unpooling: the transposed convolution whose taps are identity matrices
    d_up = rng.normal(size=(len(loc), cout)).astype(np.float32)
    got = p.unpool_bwd(out_sp, in_sp, size, stride, cout, d_up)
    yt = _t64(yc, True)
    eye = _t64(np.broadcast_to(np.eye(cout), (K, 1, cout, cout)).copy())
    up = bf._CONVT[dim](_dense_t(loc_out, yt, out_sp, batch), bf.dense_weight(eye, dim, sz).transpose(0, 1).contiguous(),
                        stride=st)
    (gy,) = _grads((_sample_t(up, loc) * _t64(d_up)).sum(), yt)
    assert_close(got, gy, "unpooling d_input")
    return p


def check_bn_train(make, seed, n=257, C=13):
    """Training-mode batch norm forward and backward (CPU/BatchNormalization.cpp:13-107)."""
    import torch
    F = torch.nn.functional
    rng = np.random.default_rng(seed)
    p = make(2)
    for leak, affine in ((0.0, True), (0.333, True), (1.0, False)):
        x = (rng.normal(size=(n, C)) * 2 + 1).astype(np.float32)
        g = rng.uniform(0.5, 1.5, C).astype(np.float32) if affine else None
        b = rng.normal(size=C).astype(np.float32) if affine else None
        rm, rv = rng.normal(size=C).astype(np.float32), rng.uniform(0.5, 1.5, C).astype(np.float32)
        out, sm, si, rm2, rv2 = p.bn_train(x, rm, rv, g, b, 1e-4, 0.9, leak)
        xt = _t64(x, True)
        gt = _t64(g, True) if affine else None
        bt = _t64(b, True) if affine else None
        trm, trv = _t64(rm), _t64(rv)
        y = F.batch_norm(xt, trm, trv, gt, bt, True, 1 - 0.9, 1e-4)
        y = torch.where(y > 0, y, y * leak)
        assert_close(out, y.detach().numpy(), "batch norm (training) output")
        assert_close(sm, x.astype(np.float64).mean(0), "saved mean")
        assert_close(si, 1 / np.sqrt(x.astype(np.float64).var(0) + 1e-4), "saved inverse std")
        assert_close(rm2, trm.numpy(), "running mean")
        assert_close(rv2, trv.numpy(), "running variance")
        d_out = rng.normal(size=(n, C)).astype(np.float32)
        # an output within rounding of zero may be on either side of the leaky ReLU's kink in fp32:
        # such values get no gradient, so that their side does not matter
        d_out[np.abs(y.detach().numpy()) < 1e-5] = 0
        d_in, d_g, d_b = p.bn_bwd(x, out, d_out, sm, si, g, leak, affine)
        gx, gg, gb = _grads((y * _t64(d_out)).sum(), xt, gt, bt)
        assert_close(d_in, gx, "batch norm d_input")
        if affine:
            assert_close(d_g, gg, "batch norm d_weight")
            assert_close(d_b, gb, "batch norm d_bias")


def check_io_backward(make, dim, mode, seed, n=300, spatial=9, batch=3, planes=4):
    """InputLayer / OutputLayer backward (CPU/IOLayers.cpp:73-93,116-135) against the rule rows."""
    rng = np.random.default_rng(seed)
    coords = bf.random_sites(rng, dim, spatial, n, batch, duplicates=0 if mode == 0 else n // 2)
    if mode == 0:
        coords = np.unique(coords, axis=0)
    p = make(dim)
    n_out = p.input_layer(spatial, coords, 0, mode)
    row_of, _ = bf.first_occurrence_rows(coords)
    d_out = rng.normal(size=(n_out, planes)).astype(np.float32)
    got = p.input_bwd(d_out)
    groups = {}
    for i, r in enumerate(row_of):
        groups.setdefault(int(r), []).append(i)
    want = np.zeros((len(coords), planes))
    for r, pts in groups.items():
        if mode in (0, 3):
            want[pts] = d_out[r]
        elif mode == 4:
            want[pts] = d_out[r].astype(np.float64) * np.float32(1.0 / len(pts))
        elif mode == 1:
            want[pts[0]] = d_out[r]
        else:
            want[pts[-1]] = d_out[r]
    assert_close(got, want, "input layer d_input, mode %d" % mode)
    d_pts = rng.normal(size=(len(coords), planes)).astype(np.float32)
    got = p.output_bwd(d_pts)
    want = np.zeros((n_out, planes))
    for r, pts in groups.items():
        listed = pts if mode in (0, 3, 4) else ([pts[0]] if mode == 1 else [pts[-1]])
        want[r] = d_pts[listed].astype(np.float64).sum(0)
    assert_close(got, want, "output layer d_input, mode %d" % mode)


def check_bl_backward(make, dim, mode, seed, batch=3, length=70, spatial=9, planes=5):
    """BLInputLayer / BLOutputLayer backward (CPU/IOLayers.cpp:161-184,207-229)."""
    rng = np.random.default_rng(seed)
    coords = rng.integers(0, spatial, (batch, length, dim)).astype(np.int64)
    if mode != 0:
        coords[rng.random((batch, length)) < 0.2] = -1
    p = make(dim)
    n_out = p.bl_input_layer(spatial, coords, mode)
    hdr, rows = p.bl_rules()
    d_out = rng.normal(size=(n_out, planes)).astype(np.float32)
    got = p.bl_input_bwd(d_out)
    want = np.zeros((batch * length, planes))
    if mode == 0:
        want[:] = d_out
    else:
        for r in range(n_out):
            cnt = rows[r, 0]
            for i in rows[r, 1:1 + cnt]:
                want[i] += d_out[r].astype(np.float64) * (np.float32(1.0 / cnt) if mode == 4 else 1.0)
    assert_close(got.reshape(-1, planes), want, "batch-by-length input d_input, mode %d" % mode)
    d_pts = rng.normal(size=(batch, length, planes)).astype(np.float32)
    got = p.bl_output_bwd(d_pts)
    flat = d_pts.reshape(-1, planes)
    want = np.zeros((n_out, planes))
    if mode == 0:
        want[:] = flat
    else:
        for r in range(n_out):
            want[r] = flat[rows[r, 1:1 + rows[r, 0]]].astype(np.float64).sum(0)
    assert_close(got, want, "batch-by-length output d_input, mode %d" % mode)


def check_misc_backward(make, seed):
    """SparseToDense and NetworkInNetwork backward (CPU/SparseToDense.cpp:21-33,66-90,
    CPU/NetworkInNetwork.cpp:24-47)."""
    rng, p, loc, x = _setup(make, 2, 6, 60, 3, seed, 4)
    d_dense = rng.normal(size=(3, 4, 6, 6)).astype(np.float32)
    got = p.s2d_bwd(6, d_dense)
    assert_close(got, bf.sample_dense(_t64(d_dense), loc), "sparse to dense d_input")
    for rows, cin, cout in ((257, 13, 7), (64, 32, 32), (300, 64, 96)):
        a = rng.normal(size=(rows, cin)).astype(np.float32)
        w = (rng.normal(size=(cin, cout)) * 0.3).astype(np.float32)
        d = rng.normal(size=(rows, cout)).astype(np.float32)
        d_in, d_w, d_b = p.nin_bwd(a, d, w, with_bias=True)
        a64, w64, d64 = a.astype(np.float64), w.astype(np.float64), d.astype(np.float64)
        assert_close(d_in, d64 @ w64.T, "network in network d_input")
        assert_close(d_w, a64.T @ d64, "network in network d_weight")
        assert_close(d_b, d64.sum(0), "network in network d_bias")
