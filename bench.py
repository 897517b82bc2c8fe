"""Benchmark of the sparse-convolution forward path on one MI355X.

Default workload ("sweep"): the single-layer configuration at scene scale - one synthetic
room of 1,000,000 active voxels in a 4096^3 grid, SubmanifoldConvolution 3^3, fp32, for
(nIn, nOut) in {(3,32), (32,32), (64,64), (128,128), (256,256)}.  One step = one forward of
each of the five convolutions with the rulebook already built (its build time is reported
separately as `rulebook_ms`).  `value` = sum of 2*MACs / sum of time, in GFLOP/s, with MACs
counted as the reference counts them (sum over filter taps of rules * nIn * nOut).

Prints ONE JSON line.  `roofline` describes the kernel that takes the largest share of the
step; `sweep` lists every channel pair with its own roofline; `cpu_baseline` times the
reference's CPU path (oracle/_ref, else the oracle port) on a bounded sample."""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
MFMA_FP32_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PAIRS = [(3, 32), (32, 32), (64, 64), (128, 128), (256, 256)]
# HBM-side bytes per launch on the default workload (1,000,000 sites, seed 3000, shuffled), from
# rocprofv3 FETCH_SIZE / WRITE_SIZE passes scaled by a 1 GiB copy kernel (x2.000 / x1.000):
# profiles/conv256_sweep1M_pmc.txt.  Only reported when the run is that workload.
MEASURED_TRAFFIC = {(256, 256): 7.70e9, (128, 128): 1.62e9, (64, 64): 0.782e9, (32, 32): 0.430e9, (3, 32): 0.501e9}


def conv_bytes(R, n_out_rows, K, cin, cout, s=4):
    """Algorithmic bytes of one convolution forward: gathered input rows + int32 rule pairs +
    output written once + weights once."""
    return R * cin * s + 8 * R + n_out_rows * cout * s + K * cin * cout * s


def roofline_for(cin, cout, R, n, K, ms, traffic=None):
    flops = 2.0 * R * cin * cout
    byts = conv_bytes(R, n, K, cin, cout)
    t_mfma = flops / (MFMA_FP32_TFLOPS * 1e12)
    t_hbm = byts / (HBM_PEAK_GBS * 1e9)
    if t_mfma >= t_hbm:
        ach = flops / (ms * 1e-3) / 1e12
        return {"bound": "mfma", "achieved": round(ach, 3), "peak": MFMA_FP32_TFLOPS, "unit": "TFLOP/s",
                "frac": round(ach / MFMA_FP32_TFLOPS, 4), "traffic": traffic}
    ach = byts / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": traffic}


def cpu_baseline(sample_sites, seed):
    """Reference CPU path (compiled reference if oracle/_ref is there, else the oracle port) on
    a smaller scene of the same generator: the same five convolutions, once each."""
    from oracle import cpu_path
    from sparseconvnet_amd import synthetic
    kind = "reference" if cpu_path.available("ref") else "port"
    flavour = "ref" if kind == "reference" else "oracle"
    if flavour == "oracle" and not cpu_path.available("oracle"):
        return None
    coords = synthetic.room_scene(seed=seed, target=sample_sites, spatial=4096)
    p = cpu_path.CpuPath(3, flavour)
    p.input_layer(4096, coords, 0, 0)
    t0 = time.time()
    rules = p.submanifold_rules(4096, 3)
    t_rules = time.time() - t0
    R = sum(len(r) for r in rules)
    rng = np.random.default_rng(0)
    flops = 0.0
    secs = 0.0
    for cin, cout in PAIRS:
        x = rng.normal(size=(len(coords), cin)).astype(np.float32)
        w = (rng.normal(size=(27, 1, cin, cout)) * (2.0 / (cin * 27)) ** 0.5).astype(np.float32)
        t0 = time.time()
        _, macs = p.subm_conv(4096, 3, x, w)
        secs += time.time() - t0
        flops += 2.0 * macs
    try:
        import torch
        cores = torch.get_num_threads() if kind == "reference" else int(os.environ.get("OMP_NUM_THREADS", os.cpu_count()))
    except Exception:
        cores = os.cpu_count()
    return {"value": round(flops / secs / 1e9, 2), "unit": "GFLOP/s", "cores": int(cores), "kind": kind,
            "sample": "same sweep of 5 SubmanifoldConvolution 3^3 forwards, once each, on a %d-site room "
                      "scene (%d rules); rulebook build %.2f s single-threaded, not included"
                      % (len(coords), R, t_rules)}


def unet_scene(sites, seed, reps=7, residual=False, batch=1):
    """3D U-Net forward of examples/ScanNet/unet.py:25-38 with m=32, block_reps=2 (7 levels,
    [32..224] planes), InputLayer mode 4 on a room scene with ~30% duplicated points, eval,
    random-init weights, batch 1.  cold = new Metadata per scene, as a user runs it (input layer,
    every rulebook and all layers); warm = the same scene again with its rulebooks cached.
    residual: the builder's ResNet-style blocks (networkArchitectures.py:222-230) instead of
    the VGG-style ones the example uses.  batch: that many scenes of `sites` sites in one call
    (examples/ScanNet/unet.py trains and validates with batches of scenes)."""
    import torch
    import sparseconvnet_amd as scn
    from sparseconvnet_amd import synthetic
    m = 32
    torch.manual_seed(0)
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 2, [m, 2 * m, 3 * m, 4 * m, 5 * m, 6 * m, 7 * m], residual)).add(
        scn.OutputLayer(3)).cuda().eval()
    linear = torch.nn.Linear(m, 20).cuda()
    if batch == 1:
        coords = synthetic.room_scene(seed=seed, target=sites, spatial=4096, duplicate_fraction=0.3)
    else:
        coords = synthetic.scene_batch(seed=seed, batch=batch, target=sites, spatial=4096, duplicate_fraction=0.3)
    g = torch.Generator(device="cuda").manual_seed(1)
    feats = torch.rand((len(coords), 3), device="cuda", generator=g) * 2 - 1
    cd = torch.as_tensor(coords).cuda()
    inp_layer = scn.InputLayer(3, 4096, mode=4)
    cold, warm = [], []
    with torch.no_grad():
        for r in range(reps + 1):
            scn.forward_pass_multiplyAdd_count = 0
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            x = inp_layer([cd, feats])
            y = linear(model(x))
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            y = linear(model(x))
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            if r:  # first pass warms allocators and code objects
                cold.append((t1 - t0) * 1e3)
                warm.append((t2 - t1) * 1e3)
            macs = scn.forward_pass_multiplyAdd_count / 2
    if batch > 1:
        return {"unet_batch%d_ms_per_batch" % batch: round(float(np.median(cold)), 3),
                "unet_batch%d_warm_ms_per_batch" % batch: round(float(np.median(warm)), 3),
                "unet_batch%d_active_sites" % batch: int(x.features.shape[0])}
    if residual:
        return {"unet_residual_ms_per_scene": round(float(np.median(cold)), 3),
                "unet_residual_warm_ms": round(float(np.median(warm)), 3),
                "unet_residual_gflop": round(2 * macs / 1e9, 2)}
    return {"unet_ms_per_scene": round(float(np.median(cold)), 3), "unet_warm_ms": round(float(np.median(warm)), 3),
            "unet_points": int(len(coords)), "unet_active_sites": int(x.features.shape[0]),
            "unet_gflop": round(2 * macs / 1e9, 2),
            "unet_warm_gflops": round(2 * macs / (float(np.median(warm)) * 1e-3) / 1e9, 1)}


def other_ops(sites, seed):
    """The rest of the path on the same kind of scene, each op by itself with inputs resident
    in HBM: ms (median of 5, HIP events on the launch stream) and the algorithmic bytes it has
    to move, against the 8 TB/s of HBM.  Rulebook builds are timed from the host (they
    synchronise)."""
    import torch
    import sparseconvnet_amd as scn
    from sparseconvnet_amd import metadata as M
    from sparseconvnet_amd import synthetic

    def timed(fn, reps=5):
        fn()
        ms = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            ms.append(e0.elapsed_time(e1))
        return float(np.median(ms))

    def host_timed(fn, reps=4):
        ms = []
        for _ in range(reps + 1):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            keep = fn()
            torch.cuda.synchronize()
            ms.append((time.perf_counter() - t0) * 1e3)
            del keep
        return float(np.median(ms[1:]))

    def row(name, ms, byts, **extra):
        d = {"op": name, "ms": round(ms, 4), "algorithmic_MB": round(byts / 1e6, 1),
             "GB_per_s": round(byts / (ms * 1e-3) / 1e9, 1), "frac_hbm": round(byts / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        d.update(extra)
        return d

    coords = synthetic.room_scene(seed=seed, target=sites, spatial=4096, duplicate_fraction=0.3)
    npts = len(coords)
    cd = torch.as_tensor(coords).cuda()
    g = torch.Generator(device="cuda").manual_seed(2)
    feats = torch.rand((npts, 3), device="cuda", generator=g)
    sz, half = torch.LongTensor([4096] * 3), torch.LongTensor([2048] * 3)
    two = torch.LongTensor([2] * 3)
    out = []

    def input_layer():
        md = M.Metadata(3)
        md.inputLayer(sz, cd, feats, 0, 4)
        return md
    ms = host_timed(input_layer)
    md = M.Metadata(3)
    x3 = md.inputLayer(sz, cd, feats, 0, 4)
    n = x3.shape[0]
    # coordinates read (4 int64 per point), level written (4 int32 + key per site), rules (2 int32 per point)
    out.append(row("InputLayer mode 4: rules + level (%d points -> %d sites)" % (npts, n), ms,
                   npts * 32 + n * 24 + npts * 8, points_per_s=round(npts / (ms * 1e-3))))
    L, stream = md._L, C.c_void_p(torch.cuda.current_stream().cuda_stream)
    y3 = torch.empty((n, 3), device="cuda")
    ms = timed(lambda: M._lib.check(L.scn_input_layer_fwd(md._h, M._ptr(feats), M._ptr(y3), 3, stream)))
    out.append(row("InputLayer forward (mean of duplicates), 3 planes", ms, npts * 12 + npts * 4 + n * 12 + n * 8))
    x32 = torch.randn((n, 32), device="cuda", generator=g)
    x64 = torch.randn((n, 64), device="cuda", generator=g)
    ms = timed(lambda: md.outputLayer(x32))
    out.append(row("OutputLayer forward, 32 planes", ms, npts * 4 + npts * 128 + n * 128))
    mean, var = torch.zeros(64, device="cuda"), torch.ones(64, device="cuda")
    ms = timed(lambda: M.batchNormEval(x64, mean, var, None, None, 1e-4, 0.0))
    out.append(row("BatchNormReLU eval (stand-alone pass), 64 planes", ms, 2 * n * 64 * 4))

    def strided():
        m2 = M.Metadata(3)
        m2.inputLayer(sz, cd, feats, 0, 4)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        M._lib.check(L.scn_md_strided_rules(m2._h, m2._s(sz), m2._s(half), m2._s(two), m2._s(two), stream))
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3, m2
    t = []
    for _ in range(4):
        dt, m2 = strided()
        t.append(dt)
        del m2
    ms = float(np.median(t[1:]))
    w_dn = torch.randn((8, 1, 32, 64), device="cuda", generator=g) * 0.1
    w_up = torch.randn((8, 1, 64, 32), device="cuda", generator=g) * 0.1
    yc, _ = md.convolution(sz, half, two, two, x32, w_dn, None)
    nc = yc.shape[0]
    # input keys read, output level written, both rule tables written (8 taps)
    out.append(row("strided rulebook 2^3 / stride 2 + output level (%d -> %d sites)" % (n, nc), ms,
                   n * 8 + nc * 24 + 8 * 4 * (n + nc) + 8 * n, sites_per_s=round(n / (ms * 1e-3))))
    ms = timed(lambda: md.convolution(sz, half, two, two, x32, w_dn, None, want_macs=False))
    out.append(row("Convolution 2^3 / stride 2, 32 -> 64", ms, n * 32 * 4 + 8 * n + nc * 64 * 4 + 8 * 32 * 64 * 4,
                   gflops=round(2.0 * n * 32 * 64 / (ms * 1e-3) / 1e9, 1)))
    ms = timed(lambda: md.deconvolution(half, sz, two, two, yc, w_up, None, want_macs=False))
    out.append(row("Deconvolution 2^3 / stride 2, 64 -> 32", ms, nc * 64 * 4 + 8 * n + n * 32 * 4 + 8 * 64 * 32 * 4,
                   gflops=round(2.0 * n * 64 * 32 / (ms * 1e-3) / 1e9, 1)))
    w_nin = torch.randn((64, 32), device="cuda", generator=g) * 0.1
    ms = timed(lambda: md.networkInNetwork(x64, w_nin, None, want_macs=False))
    out.append(row("NetworkInNetwork 64 -> 32", ms, n * 64 * 4 + n * 32 * 4 + 64 * 32 * 4,
                   gflops=round(2.0 * n * 64 * 32 / (ms * 1e-3) / 1e9, 1)))
    ms = timed(lambda: md.maxPooling(sz, half, two, two, x32, 0))
    out.append(row("MaxPooling 2^3 / stride 2, 32 planes", ms, n * 32 * 4 + 8 * n + nc * 32 * 4))
    ms = timed(lambda: md.averagePooling(sz, half, two, two, x32, 0))
    out.append(row("AveragePooling 2^3 / stride 2, 32 planes", ms, n * 32 * 4 + 8 * n + nc * 32 * 4))
    xc32 = torch.randn((nc, 32), device="cuda", generator=g)
    ms = timed(lambda: md.unPooling(half, sz, two, two, xc32, 0))
    out.append(row("UnPooling 2^3 / stride 2, 32 planes", ms, nc * 32 * 4 + 8 * n + n * 32 * 4))

    # the other two input routes on the same points: batch-by-length (one sample, every position
    # filled) and the point-at-a-time batch with a third of its points overwriting
    cbl = cd[:, :3].reshape(1, npts, 3).contiguous()
    fbl = feats.reshape(1, npts, 3)

    def bl_layer():
        m3 = M.Metadata(3)
        m3.blInputLayer(sz, cbl, fbl, 4)
        return m3
    ms = host_timed(bl_layer)
    out.append(row("BLInputLayer mode 4: rules + level + forward (%d points)" % npts, ms,
                   npts * 24 + n * 24 + npts * 8 + npts * 12 + n * 12, points_per_s=round(npts / (ms * 1e-3))))
    flags = (torch.arange(npts, device="cuda") % 3 == 0).to(torch.uint8)

    def input_batch():
        m3 = M.Metadata(3)
        m3.inputBatch(sz, cd, feats, flags, 1)
        return m3
    ms = host_timed(input_batch)
    out.append(row("InputBatch (a third of the points overwrite): level + features (%d points)" % npts, ms,
                   npts * 33 + n * 24 + npts * 8 + npts * 12 + n * 12, points_per_s=round(npts / (ms * 1e-3))))

    def chain():
        m3 = M.Metadata(3)
        m3.inputLayer(sz, cd, feats, 0, 4)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        m3.generateRuleBooks2s2()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3, m3
    t = []
    for _ in range(4):
        dt, m3 = chain()
        t.append(dt)
        levels = [m3.getNActive(torch.LongTensor([4096 >> l] * 3)) for l in range(13)]
        del m3
    ms = float(np.median(t[1:]))
    total = sum(levels)
    # per level: keys read, 27-tap table written, the strided pair of tables and the next level written
    out.append(row("precompute_metadata(2): 3^3 and 2^3/stride-2 rulebooks of all %d levels (%d sites in all)"
                   % (sum(1 for v in levels if v), total), ms, total * (8 + 27 * 4 + 24 + 2 * 8 * 4),
                   sites_per_s=round(total / (ms * 1e-3))))
    # sparse to dense on a grid that can be dense: the same scene generator at 128^3, 16 planes
    c2 = synthetic.room_scene(seed=seed + 1, target=200000, spatial=128)
    md2 = M.Metadata(3)
    s128 = torch.LongTensor([128] * 3)
    f2 = torch.randn((len(c2), 16), device="cuda", generator=g)
    xs = md2.inputLayer(s128, torch.as_tensor(c2).cuda(), f2, 0, 3)
    ms = timed(lambda: md2.sparseToDense(s128, xs, 16))
    out.append(row("SparseToDense 128^3, 16 planes (%d sites)" % xs.shape[0], ms, xs.shape[0] * 16 * 4 + 128 ** 3 * 16 * 4))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--sites", type=int, default=1000000)
    ap.add_argument("--seed", type=int, default=3000)
    ap.add_argument("--order", default="shuffled", choices=["shuffled", "scan"])
    ap.add_argument("--cpu-sites", type=int, default=1000000)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--pairs", default="")
    ap.add_argument("--no-unet", action="store_true")
    ap.add_argument("--no-ops", action="store_true")
    ap.add_argument("--no-bf16", action="store_true")
    ap.add_argument("--no-residual", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy 3 times, to scale profiler byte counters")
    ap.add_argument("--unet-sites", type=int, default=1000000)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU; this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    from sparseconvnet_amd import _lib, synthetic
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    L = _lib.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    pairs = PAIRS if not args.pairs else [tuple(int(v) for v in p.split("x")) for p in args.pairs.split(",")]

    coords = synthetic.room_scene(seed=args.seed, target=args.sites, spatial=4096, order=args.order)
    cd = torch.as_tensor(coords).cuda()
    sp, fs = _lib.sizes(3, 4096), _lib.sizes(3, 3)

    def build():
        h = L.scn_md_create(3)
        n = C.c_int64(0)
        _lib.check(L.scn_md_input_layer(h, sp, C.c_void_p(cd.data_ptr()), len(coords), 4, 0, 0, stream,
                                        C.byref(n)))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        _lib.check(L.scn_md_submanifold_rules(h, sp, fs, stream))
        torch.cuda.synchronize()
        return h, int(n.value), (time.perf_counter() - t0) * 1e3

    rb_ms = []
    for _ in range(4):
        h, n, ms = build()
        rb_ms.append(ms)
        L.scn_md_destroy(h)
    h, n, ms = build()
    rb_ms.append(ms)
    rulebook_ms = float(np.median(rb_ms[1:]))
    sizes = (C.c_int64 * 27)()
    _lib.check(L.scn_rules_sizes(h, 0, sp, fs, None, None, stream, sizes))
    R = int(sum(sizes))

    g = torch.Generator(device="cuda").manual_seed(0)
    work = []
    for cin, cout in pairs:
        x = torch.randn((n, cin), device="cuda", generator=g)
        w = torch.randn((27, 1, cin, cout), device="cuda", generator=g) * (2.0 / (cin * 27)) ** 0.5
        y = torch.empty((n, cout), device="cuda")
        work.append((cin, cout, x, w, y))

    macs = C.c_double(0)

    def conv(cin, cout, x, w, y):
        _lib.check(L.scn_subm_conv_fwd(h, sp, fs, C.c_void_p(x.data_ptr()), C.c_void_p(y.data_ptr()),
                                       C.c_void_p(w.data_ptr()), None, cin, cout, 1, stream, C.byref(macs)))

    for _ in range(args.warmup):
        for wk in work:
            conv(*wk)
    torch.cuda.synchronize()
    ev = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in work]
          for _ in range(args.steps)]
    t0 = time.perf_counter()
    for s in range(args.steps):
        for i, wk in enumerate(work):
            ev[s][i][0].record()
            conv(*wk)
            ev[s][i][1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    per_pair_ms = [float(np.mean([ev[s][i][0].elapsed_time(ev[s][i][1]) for s in range(args.steps)]))
                   for i in range(len(work))]
    total_flops = sum(2.0 * R * cin * cout for cin, cout in pairs)
    value = total_flops / (ms_per_step * 1e-3) / 1e9

    default_workload = args.sites == 1000000 and args.seed == 3000 and args.order == "shuffled"
    sweep = []
    for (cin, cout), ms in zip(pairs, per_pair_ms):
        sweep.append({"nIn": cin, "nOut": cout, "ms": round(ms, 4),
                      "gflops": round(2.0 * R * cin * cout / (ms * 1e-3) / 1e9, 1),
                      "sites_per_s": round(n / (ms * 1e-3)),
                      "roofline": roofline_for(cin, cout, R, n, 27, ms,
                                               MEASURED_TRAFFIC.get((cin, cout)) if default_workload else None)})
    dom = int(np.argmax(per_pair_ms))
    roof = dict(sweep[dom]["roofline"])
    roof["kernel"] = "submanifold conv %d->%d" % pairs[dom]

    out = {
        "metric": "SubmanifoldConv GFLOP/s & % roofline; 3D U-Net ms/scene at 1 GPU",
        "value": round(value, 1), "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[2]: 3D single-layer sweep, SubmanifoldConvolution 3^3 on one "
                               "%d-voxel room scene in 4096^3 (%s point order), (nIn,nOut) in %s, "
                               "rulebook warm" % (n, args.order, pairs),
                   "active_sites": n, "rules": R},
        "rulebook_ms": round(rulebook_ms, 3),
        "rulebook_sites_per_s": round(n / (rulebook_ms * 1e-3)),
        "roofline": roof, "sweep": sweep,
    }
    if not args.no_bf16:
        # Optional reduced-precision path (bf16 operands, fp32 accumulation), same work, listed
        # beside the fp32 sweep; `value` and `roofline` above are fp32 only.
        _lib.check(L.scn_md_set_bf16(h, 1))
        wide = [(i, wk) for i, wk in enumerate(work) if wk[0] >= 32]
        for _, wk in wide:
            conv(*wk)
        torch.cuda.synchronize()
        bf = []
        for i, wk in wide:
            t = []
            for _ in range(max(2, min(args.steps, 5))):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                conv(*wk)
                e1.record()
                torch.cuda.synchronize()
                t.append(e0.elapsed_time(e1))
            ms = float(np.mean(t))
            bf.append({"nIn": wk[0], "nOut": wk[1], "ms": round(ms, 4),
                       "gflops": round(2.0 * R * wk[0] * wk[1] / (ms * 1e-3) / 1e9, 1),
                       "speedup_vs_f32": round(per_pair_ms[i] / ms, 2)})
        out["sweep_bf16"] = bf
        _lib.check(L.scn_md_set_bf16(h, 0))
    L.scn_md_destroy(h)
    del work
    if args.calibrate_copy:
        a = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b
    if not args.no_ops:
        out["other_ops"] = other_ops(args.unet_sites, 5000)
    if not args.no_unet:
        out["unet"] = unet_scene(args.unet_sites, 5000)
        if not args.no_residual:
            out["unet"].update(unet_scene(args.unet_sites, 5000, residual=True))
            out["unet"].update(unet_scene(args.unet_sites, 7000, reps=2, batch=4))
        if not args.no_bf16:
            import sparseconvnet_amd as scn
            scn.bf16_mfma = True
            u = unet_scene(args.unet_sites, 5000)
            scn.bf16_mfma = False
            out["unet"].update({"unet_bf16_ms_per_scene": u["unet_ms_per_scene"], "unet_bf16_warm_ms": u["unet_warm_ms"]})
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.cpu_sites, args.seed)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
