"""Writes the golden fixtures in this directory from the compiled reference
(oracle/_ref/libscn_ref.so, built by oracle/Makefile where the reference tree
is present).  Run from the repository root:  python tests/golden/make_golden.py

Every fixture is data only: seeded inputs plus what the reference computed for
them, stored in canonical form (rulebooks as sorted (offset, in-site, out-site)
rows; feature matrices with rows sorted by (sample, coordinates)) so that they
do not depend on how an implementation numbers its rows.  Each writer takes
`make(dim)` returning an object with oracle.cpu_path.CpuPath's interface, so the
tests run the same recipe on the implementation under test and compare files."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle.cpu_path import CpuPath, canon_rows, canon_rules  # noqa: E402
from sparseconvnet_amd import synthetic  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def canon_feats(loc, x):
    return x[canon_rows(loc)]


def single_layer(path, make):
    """Configuration-1 shape at 32^3: batch 2, SubmanifoldConvolution 3^3 16->16, no bias."""
    rng = np.random.default_rng(101)
    coords = synthetic.config1(seed=1000, batch=2, spatial=32, target=700)
    feats = rng.normal(size=(len(coords), 16)).astype(np.float32)
    w = (rng.normal(size=(27, 1, 16, 16)) * (2.0 / (16 * 27)) ** 0.5).astype(np.float32)
    p = make(3)
    p.input_layer(32, coords, 0, 0)
    loc = p.spatial_locations(32)
    rules = p.submanifold_rules(32, 3)
    y, macs = p.subm_conv(32, 3, feats, w)
    np.savez_compressed(path, coords=coords, feats=feats, w=w, loc=loc,
                        rules=canon_rules(rules, loc, loc).astype(np.int16),
                        y=canon_feats(loc, y), macs=macs)


def strided_tree(path, make):
    """Configuration-4 shape at 62^3: h=Conv(2,2)(x); p=MaxPool(3,2)(h); u=Deconv(2,2)(h);
    y=BatchNormReLU(u).  InputLayer mode 4 with duplicated points."""
    rng = np.random.default_rng(104)
    coords = synthetic.room_scene(seed=4000, target=1500, spatial=62, n_boxes=6,
                                  duplicate_fraction=0.3)
    feats = rng.uniform(-1, 1, size=(len(coords), 8)).astype(np.float32)
    w1 = (rng.normal(size=(8, 1, 8, 12)) * 0.2).astype(np.float32)
    w2 = (rng.normal(size=(8, 1, 12, 8)) * 0.2).astype(np.float32)
    mean = rng.normal(size=8).astype(np.float32)
    var = rng.uniform(0.5, 1.5, 8).astype(np.float32)
    gamma = rng.normal(size=8).astype(np.float32)
    beta = rng.normal(size=8).astype(np.float32)
    p = make(3)
    p.input_layer(62, coords, 0, 4)
    loc0 = p.spatial_locations(62)
    x = p.input_fwd(feats)
    r_conv = p.strided_rules(62, 31, 2, 2)
    loc1 = p.spatial_locations(31)
    h, macs1 = p.conv(62, 31, 2, 2, x, w1)
    r_pool = p.strided_rules(31, 15, 3, 2)
    loc2 = p.spatial_locations(15)
    pooled = p.maxpool(31, 15, 3, 2, h)
    u, macs2 = p.deconv(31, 62, 2, 2, h, w2)
    y = p.bn_eval(u, mean, var, gamma, beta, 1e-4, 0.0)
    back = p.output_fwd(y)
    np.savez_compressed(
        path, coords=coords, feats=feats, w1=w1, w2=w2, mean=mean, var=var, gamma=gamma, beta=beta,
        loc0=loc0[canon_rows(loc0)], x=canon_feats(loc0, x),
        rules_conv=canon_rules(r_conv, loc0, loc1).astype(np.int16),
        loc1=loc1[canon_rows(loc1)], h=canon_feats(loc1, h), macs1=macs1,
        rules_pool=canon_rules(r_pool, loc1, loc2).astype(np.int16),
        loc2=loc2[canon_rows(loc2)], pooled=canon_feats(loc2, pooled),
        u=canon_feats(loc0, u), macs2=macs2, y=canon_feats(loc0, y), back=back)


def vgg2d(path, make):
    """Configuration-2 shape with 4 samples in a 31x31 grid: SC 1->8, BNReLU, MP3/2,
    SC 8->16, BNReLU, MP3/2, SparseToDense (output 7x7)."""
    rng = np.random.default_rng(102)
    coords = synthetic.strokes2d(seed=2000, batch=4, canvas=28, spatial=31)
    feats = np.ones((len(coords), 1), np.float32)
    w1 = (rng.normal(size=(9, 1, 1, 8)) * (2.0 / 9) ** 0.5).astype(np.float32)
    w2 = (rng.normal(size=(9, 1, 8, 16)) * (2.0 / 72) ** 0.5).astype(np.float32)
    bn1 = [rng.normal(size=8).astype(np.float32), rng.uniform(0.5, 1.5, 8).astype(np.float32)]
    bn2 = [rng.normal(size=16).astype(np.float32), rng.uniform(0.5, 1.5, 16).astype(np.float32)]
    p = make(2)
    p.input_layer(31, coords, 0, 3)
    x = p.input_fwd(feats)
    a, _ = p.subm_conv(31, 3, x, w1)
    a = p.bn_eval(a, bn1[0], bn1[1], None, None, 1e-4, 0.0)
    a = p.maxpool(31, 15, 3, 2, a)
    a, _ = p.subm_conv(15, 3, a, w2)
    a = p.bn_eval(a, bn2[0], bn2[1], None, None, 1e-4, 0.0)
    a = p.maxpool(15, 7, 3, 2, a)
    dense = p.s2d(7, a)
    np.savez_compressed(path, coords=coords, feats=feats, w1=w1, w2=w2, bn1_mean=bn1[0],
                        bn1_var=bn1[1], bn2_mean=bn2[0], bn2_var=bn2[1], dense=dense)


def residual_block(path, make):
    """One residual block of the U-Net builder (networkArchitectures.py:222-230) at 24^3,
    6 -> 10 planes: NetworkInNetwork(x) + SC(BNReLU(SC(BNReLU(x)))), and a second
    NetworkInNetwork with bias on the sum."""
    rng = np.random.default_rng(106)
    coords = synthetic.config1(seed=6000, batch=2, spatial=24, target=500)
    feats = rng.normal(size=(len(coords), 6)).astype(np.float32)
    wn = (rng.normal(size=(6, 10)) * (2.0 / 6) ** 0.5).astype(np.float32)
    w1 = (rng.normal(size=(27, 1, 6, 10)) * (2.0 / (6 * 27)) ** 0.5).astype(np.float32)
    w2 = (rng.normal(size=(27, 1, 10, 10)) * (2.0 / (10 * 27)) ** 0.5).astype(np.float32)
    wn2 = (rng.normal(size=(10, 4)) * (2.0 / 10) ** 0.5).astype(np.float32)
    bias2 = rng.normal(size=4).astype(np.float32)
    bn1 = [rng.normal(size=6).astype(np.float32), rng.uniform(0.5, 1.5, 6).astype(np.float32)]
    bn2 = [rng.normal(size=10).astype(np.float32), rng.uniform(0.5, 1.5, 10).astype(np.float32)]
    p = make(3)
    p.input_layer(24, coords, 0, 0)
    loc = p.spatial_locations(24)
    skip, macs_nin = p.nin(feats, wn)
    a = p.bn_eval(feats, bn1[0], bn1[1], None, None, 1e-4, 0.0)
    a, _ = p.subm_conv(24, 3, a, w1)
    a = p.bn_eval(a, bn2[0], bn2[1], None, None, 1e-4, 0.0)
    a, _ = p.subm_conv(24, 3, a, w2)
    y = skip + a
    z, _ = p.nin(y, wn2, bias2)
    np.savez_compressed(path, coords=coords, feats=feats, wn=wn, w1=w1, w2=w2, wn2=wn2, bias2=bias2,
                        bn1_mean=bn1[0], bn1_var=bn1[1], bn2_mean=bn2[0], bn2_var=bn2[1],
                        skip=canon_feats(loc, skip), macs_nin=macs_nin, y=canon_feats(loc, y),
                        z=canon_feats(loc, z))


FIXTURES = {"single_layer_32.npz": single_layer, "strided_tree_62.npz": strided_tree,
            "vgg2d_31.npz": vgg2d, "residual_block_24.npz": residual_block}

if __name__ == "__main__":
    ref = lambda dim: CpuPath(dim, "ref")  # noqa: E731
    for name, fn in FIXTURES.items():
        fn(os.path.join(HERE, name), ref)
    for f in sorted(os.listdir(HERE)):
        print(f, os.path.getsize(os.path.join(HERE, f)))
