"""Benchmark of the sparse-convolution forward path on one MI355X.

Default workload ("sweep"): the single-layer configuration at scene scale - one synthetic
room of 1,000,000 active voxels in a 4096^3 grid, SubmanifoldConvolution 3^3, fp32, for
(nIn, nOut) in {(3,32), (32,32), (64,64), (128,128), (256,256)}.  One step = one forward of
each of the five convolutions with the rulebook already built (its build time is reported
separately as `rulebook_ms`).  `value` = sum of 2*MACs / sum of time, in GFLOP/s, with MACs
counted as the reference counts them (sum over filter taps of rules * nIn * nOut).

Prints ONE JSON line.  `roofline` describes the kernel that takes the largest share of the
step; `sweep` lists every channel pair with its own roofline; `cpu_baseline` times the
reference's CPU path (oracle/_ref, else the oracle port) on a bounded sample; `configs` holds
the other benchmark configurations at their own shapes."""
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
MFMA_BF16_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak
PAIRS = [(3, 32), (32, 32), (64, 64), (128, 128), (256, 256)]
TRAFFIC_FILE = os.path.join("profiles", "conv_sweep1M_pmc.txt")


def measured_traffic():
    """HBM-side bytes per launch of the sweep's kernels on the default workload, read from the
    committed counter summary (rocprofv3 FETCH_SIZE / WRITE_SIZE passes scaled by a plain copy
    of known size; the file gives the commands).  Lines `nIn nOut kernel GB` after the line
    `traffic_per_launch`.  Nothing is typed in here: without the file the field is null."""
    out = {}
    path = os.path.join(ROOT, TRAFFIC_FILE)
    if not os.path.exists(path):
        return out
    seen = False
    for line in open(path):
        if line.startswith("traffic_per_launch"):
            seen = True
            continue
        f = line.split()
        if seen and len(f) == 4 and f[0].isdigit() and f[1].isdigit():
            out[(int(f[0]), int(f[1]))] = (float(f[3]) * 1e9, f[2])
    return out


def hbm_roofline(byts, ms):
    ach = byts / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(ach / HBM_PEAK_GBS, 4), "algorithmic_MB": round(byts / 1e6, 1)}


def subm_rulebook_bytes(N, K, R):
    """Submanifold rulebook build: packed keys read, table written and read back (12 bytes per
    entry at load 0.5), one 12-byte probe per neighbour, 8 bytes per rule out."""
    return N * 8 + 2 * N * 12 / 0.5 + K * N * 12 + 8 * R


def strided_rulebook_bytes(N, N_out, R):
    return N * 8 + (N + N_out) * 12 / 0.5 + 8 * R + N_out * 8


def conv_bytes(R, n_out_rows, K, cin, cout, s=4):
    """Algorithmic bytes of one convolution forward: gathered input rows + int32 rule pairs +
    output written once + weights once."""
    return R * cin * s + 8 * R + n_out_rows * cout * s + K * cin * cout * s


def roofline_for(cin, cout, R, n, K, ms, traffic=None):
    """traffic: (bytes, kernel name) from the committed counter summary, or None."""
    flops = 2.0 * R * cin * cout
    byts = conv_bytes(R, n, K, cin, cout)
    t_mfma = flops / (MFMA_FP32_TFLOPS * 1e12)
    t_hbm = byts / (HBM_PEAK_GBS * 1e9)
    tr = {"traffic": traffic[0] if traffic else None}
    if traffic:
        tr["traffic_source"] = {"file": TRAFFIC_FILE, "kernel": traffic[1]}
    if t_mfma >= t_hbm:
        ach = flops / (ms * 1e-3) / 1e12
        return dict({"bound": "mfma", "achieved": round(ach, 3), "peak": MFMA_FP32_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(ach / MFMA_FP32_TFLOPS, 4)}, **tr)
    ach = byts / (ms * 1e-3) / 1e9
    return dict({"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                 "frac": round(ach / HBM_PEAK_GBS, 4)}, **tr)


def gpu_outputs(coords, work):
    """The library's outputs for the CPU leg's own inputs: rows in the order of the points (input
    mode 0 on distinct points), one SubmanifoldConvolution 3^3 per (x, w) of `work`."""
    import torch
    from sparseconvnet_amd import _lib
    L = _lib.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    sp, fs = _lib.sizes(3, 4096), _lib.sizes(3, 3)
    cd = torch.as_tensor(coords).cuda()
    h = L.scn_md_create(3)
    n = C.c_int64(0)
    _lib.check(L.scn_md_input_layer(h, sp, C.c_void_p(cd.data_ptr()), len(coords), coords.shape[1], 0, 0, stream,
                                    C.byref(n)))
    assert n.value == len(coords)
    macs = C.c_double(0)
    for x, w in work:
        xd, wd = torch.as_tensor(x).cuda(), torch.as_tensor(w).cuda()
        y = torch.empty((len(coords), w.shape[-1]), device="cuda")
        _lib.check(L.scn_subm_conv_fwd(h, sp, fs, C.c_void_p(xd.data_ptr()), C.c_void_p(y.data_ptr()),
                                       C.c_void_p(wd.data_ptr()), None, x.shape[1], w.shape[-1], 1, stream,
                                       C.byref(macs)))
        yield y.cpu().numpy()
    L.scn_md_destroy(h)


def roofline_bf16(cin, cout, R, n, K, ms):
    """The bf16-operand path (rows and weights rounded to bf16 on the way into the MFMA, fp32 rows
    in memory and fp32 accumulation): same algorithmic bytes as fp32, priced against the dense
    bf16 MFMA peak or HBM, whichever bounds it."""
    flops = 2.0 * R * cin * cout
    byts = conv_bytes(R, n, K, cin, cout)
    if flops / (MFMA_BF16_TFLOPS * 1e12) >= byts / (HBM_PEAK_GBS * 1e9):
        ach = flops / (ms * 1e-3) / 1e12
        return {"bound": "mfma", "achieved": round(ach, 3), "peak": MFMA_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": round(ach / MFMA_BF16_TFLOPS, 4), "traffic": None}
    return dict(hbm_roofline(byts, ms), traffic=None)


def cpu_baseline(kind, sample_sites, seed, passes=3, compare=None):
    """The CPU path on the GPU box's host cores: the same five convolutions on a room scene of
    the same generator, one warm-up pass and the median of `passes`; the rulebook build is timed
    by itself.  kind "reference": the reference's own CPU sources compiled behind
    oracle/ref_harness.cpp (oracle/_ref); "port": this repository's restatement (oracle/).
    compare: a function (coords, work) yielding the library's output per pair; the largest
    absolute difference from the CPU outputs of the last pass is reported per pair, beside the
    largest absolute CPU output (fp32 sums of up to 27 x nIn products in a different order)."""
    from oracle import cpu_path
    from sparseconvnet_amd import synthetic
    flavour = "ref" if kind == "reference" else "oracle"
    if not cpu_path.available(flavour):
        return None
    coords = synthetic.room_scene(seed=seed, target=sample_sites, spatial=4096)
    t_rules = []
    for _ in range(2):  # the second build is the warmed one
        p = cpu_path.CpuPath(3, flavour)
        p.input_layer(4096, coords, 0, 0)
        t0 = time.time()
        rules = p.submanifold_rules(4096, 3)
        t_rules.append(time.time() - t0)
    R = sum(len(r) for r in rules)
    rng = np.random.default_rng(0)
    work = []
    for cin, cout in PAIRS:
        x = rng.normal(size=(len(coords), cin)).astype(np.float32)
        w = (rng.normal(size=(27, 1, cin, cout)) * (2.0 / (cin * 27)) ** 0.5).astype(np.float32)
        work.append((x, w))
    secs, flops, outs = [], 0.0, []
    for rep in range(passes + 1):
        t0 = time.time()
        flops, outs = 0.0, []
        for x, w in work:
            y, macs = p.subm_conv(4096, 3, x, w)
            flops += 2.0 * macs
            outs.append(y if compare is not None else None)
        if rep:
            secs.append(time.time() - t0)
    sec = float(np.median(secs))
    parity = None
    if compare is not None:
        parity = {}
        for (cin, cout), want, got in zip(PAIRS, outs, compare(coords, work)):
            parity["%dx%d" % (cin, cout)] = {"max_abs_err": float(np.abs(got - want).max()),
                                             "max_abs_out": float(np.abs(want).max())}
        del outs
    try:
        import torch
        cores = torch.get_num_threads() if kind == "reference" else int(os.environ.get("OMP_NUM_THREADS", os.cpu_count()))
    except Exception:
        cores = os.cpu_count()
    return {"value": round(flops / sec / 1e9, 2), "unit": "GFLOP/s", "cores": int(cores), "kind": kind,
            "rulebook_s": round(t_rules[-1], 3), "rulebook_cores": 1, "seconds_per_pass": round(sec, 3),
            "parity_max_err": parity,
            "sample": "the sweep's 5 SubmanifoldConvolution 3^3 forwards on a %d-site room scene (%d rules), "
                      "1 warm-up pass + median of %d; rulebook build (one sample: single-threaded in the "
                      "reference) timed by itself, second of two builds" % (len(coords), R, passes)}


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
    host_coords = torch.as_tensor(coords)  # a CPU LongTensor: what the reference's InputLayer is handed (ioLayers.py:51-65)
    cd = host_coords.cuda()
    inp_layer = scn.InputLayer(3, 4096, mode=4)
    cold, warm, cold_host = [], [], []
    scn.forward_pass_multiplyAdd_count = 0
    with torch.no_grad():
        for r in range(reps + 1):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            x = inp_layer([cd, feats])
            y = linear(model(x))
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            y = linear(model(x))
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            x = inp_layer([host_coords, feats])  # the previous scene's Metadata dies here, unsynchronised
            y = linear(model(x))
            torch.cuda.synchronize()
            t3 = time.perf_counter()
            if r:  # first pass warms allocators and code objects
                cold.append((t1 - t0) * 1e3)
                warm.append((t2 - t1) * 1e3)
                cold_host.append((t3 - t2) * 1e3)
    macs = scn.forward_pass_multiplyAdd_count / (3 * (reps + 1))
    med = lambda v: round(float(np.median(v)), 3)
    graph_ms = None
    if batch == 1 and not residual:
        # The warm forward pass captured once as a HIP graph and replayed: the same kernels without
        # the host's per-call work between them (what a serving loop over a fixed scene would run).
        side = torch.cuda.Stream()
        with torch.no_grad():
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                linear(model(x))
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                yg = linear(model(x))
            reps_ms = []
            for _ in range(reps):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                graph.replay()
                torch.cuda.synchronize()
                reps_ms.append((time.perf_counter() - t0) * 1e3)
            same = bool(torch.equal(yg, linear(model(x))))
            torch.cuda.synchronize()
        graph_ms = med(reps_ms) if same else None
        del graph
    layers = None
    if batch == 1 and not residual:
        layers = unet_layer_table(torch, scn, model, x)
    # device memory the library itself holds (rulebooks of the live handles, scratch, idle blocks of
    # its cache; features and weights are torch's): high-water mark since the process started
    import ctypes
    peak = ctypes.c_int64(0)
    scn.metadata._lib.lib().scn_cache_stats(None, None, ctypes.byref(peak), None)
    if batch > 1:
        return {"unet_batch%d_ms_per_batch" % batch: med(cold), "unet_batch%d_warm_ms_per_batch" % batch: med(warm),
                "unet_batch%d_from_host_coords_ms_per_batch" % batch: med(cold_host),
                "unet_batch%d_active_sites" % batch: int(x.features.shape[0]),
                "library_peak_MiB_after_batch%d" % batch: round(peak.value / 2 ** 20)}
    if residual:
        return {"unet_residual_ms_per_scene": med(cold), "unet_residual_warm_ms": med(warm),
                "unet_residual_gflop": round(2 * macs / 1e9, 2)}
    return {"unet_layers": layers, "unet_conv_ms_sum": round(sum(r["ms"] for r in layers), 4),
            "unet_ms_per_scene": med(cold), "unet_ms_per_scene_from_host_coords": med(cold_host),
            "unet_warm_ms": med(warm), "unet_warm_graph_replay_ms": graph_ms, "unet_points": int(len(coords)), "unet_active_sites": int(x.features.shape[0]),
            "unet_gflop": round(2 * macs / 1e9, 2), "library_peak_MiB": round(peak.value / 2 ** 20),
            "unet_warm_gflops": round(2 * macs / (float(np.median(warm)) * 1e-3) / 1e9, 1),
            "unet_warm_frac_mfma_fp32": round(2 * macs / (float(np.median(warm)) * 1e-3) / 1e12 / MFMA_FP32_TFLOPS, 4),
            "note": "ms_per_scene: new Metadata per scene (input layer, every rulebook, all layers), coordinates "
                    "resident in HBM; from_host_coords: the same with the coordinates handed over as a CPU "
                    "LongTensor (host-to-device copy inside the timed region); warm: rulebooks cached; "
                    "warm_graph_replay: the warm pass replayed as one HIP graph (null if the replay's result differed)"}


def unet_layer_table(torch, scn, model, x, reps=5):
    """Every convolution of one warm U-Net pass, in call order: HIP events on the launch stream
    around each call (median of `reps` passes), the kernel the library chose, the layer's
    multiply-adds as the reference counts them and its roofline (fp32 MFMA peak or HBM,
    whichever bounds the layer)."""
    from sparseconvnet_amd import metadata as M
    recs = []
    orig = M.Metadata._conv

    def timed_conv(self, kind, size_args, n_rows, features, weight, bias, bn, post, want_macs, out=None, second=None):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        out, macs = orig(self, kind, size_args, n_rows, features, weight, bias, bn, post, True, out, second)
        e1.record()
        kernel = self._L.scn_md_last_conv_kernel(self._h).decode()
        recs.append((kind, features.shape[0], n_rows, weight.shape[0], weight.shape[1] * weight.shape[2],
                     weight.shape[1] * weight.shape[3], macs, bn is not None, post is not None, kernel, e0, e1))
        return out, (macs if want_macs else None)
    M.Metadata._conv = timed_conv
    passes = []
    try:
        with torch.no_grad():
            for _ in range(reps + 1):
                recs.clear()
                model(x)
                torch.cuda.synchronize()
                passes.append([r[-2].elapsed_time(r[-1]) for r in recs])
    finally:
        M.Metadata._conv = orig
    ms = np.median(np.array(passes[1:]), axis=0)
    rows = []
    for r, t in zip(recs, ms):
        kind, n_in_rows, n_out_rows, K, cin, cout, macs, pre, post, kernel = r[:10]
        R = macs / (cin * cout)
        rows.append({"op": ("SubmanifoldConvolution", "Convolution", "Deconvolution")[kind],
                     "rows_in": int(n_in_rows), "rows_out": int(n_out_rows), "taps": int(K), "rules": int(R),
                     "nIn": int(cin), "nOut": int(cout), "bn_in_front": bool(pre), "bn_behind": bool(post),
                     "kernel": kernel, "ms": round(float(t), 4),
                     "tflops": round(2.0 * macs / (float(t) * 1e-3) / 1e12, 2),
                     "roofline": roofline_for(cin, cout, R, n_out_rows, K, float(t))})
    return rows


def unet_train_step(sites, seed, reps=3):
    """One training step of the same U-Net (train mode: batch norms take batch statistics) on one
    room scene: InputLayer, forward, a scalar loss, backward through every layer down to the
    input features and every parameter.  New Metadata per step, as a training loop runs."""
    import torch
    import sparseconvnet_amd as scn
    from sparseconvnet_amd import synthetic
    m = 32
    torch.manual_seed(0)
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 2, [m, 2 * m, 3 * m, 4 * m, 5 * m, 6 * m, 7 * m], False)).add(
        scn.BatchNormReLU(m)).add(scn.OutputLayer(3)).cuda().train()
    linear = torch.nn.Linear(m, 20).cuda()
    coords = synthetic.room_scene(seed=seed, target=sites, spatial=4096, duplicate_fraction=0.3)
    g = torch.Generator(device="cuda").manual_seed(1)
    feats = (torch.rand((len(coords), 3), device="cuda", generator=g) * 2 - 1).requires_grad_(True)
    cd = torch.as_tensor(coords).cuda()
    inp_layer = scn.InputLayer(3, 4096, mode=4)
    ms = []
    for r in range(reps + 1):
        for p in list(model.parameters()) + list(linear.parameters()):
            p.grad = None
        feats.grad = None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        y = linear(model(inp_layer([cd, feats])))
        y.square().mean().backward()
        torch.cuda.synchronize()
        ms.append((time.perf_counter() - t0) * 1e3)
    return {"unet_train_step_ms": round(float(np.median(ms[1:])), 3),
            "unet_train_step_note": "forward in train mode + backward of one %d-point scene, new Metadata per step, "
                                    "optimizer step not included" % len(coords)}


def _timed(torch, fn, reps=5):
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


def _host_timed(torch, fn, reps=4):
    """fn() -> (milliseconds measured inside, object to keep alive until timing ends)."""
    t = []
    for _ in range(reps + 1):
        dt, keep = fn()
        t.append(dt)
        del keep
    return float(np.median(t[1:]))


def config_rows():
    """The other benchmark configurations at their own shapes: configuration 1 (the reference's
    CPU-runnable single layer), configuration 2 (2-D VGG inference, batch 100) and configuration
    4 (the strided tree at 4094^3).  Rulebook builds are timed from the host and listed apart
    from the feature passes (HIP events on the launch stream)."""
    import torch
    import sparseconvnet_amd as scn
    from sparseconvnet_amd import metadata as M
    from sparseconvnet_amd import synthetic
    L, stream = M._lib.lib(), C.c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator(device="cuda").manual_seed(4)
    rows = {}

    def sync_ms(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3

    # configuration 1: batch 2, 128^3, ~40k sites per sample, SubmanifoldConvolution 16 -> 16
    coords = synthetic.config1()
    cd = torch.as_tensor(coords).cuda()
    s128, three = torch.LongTensor([128] * 3), torch.LongTensor([3] * 3)
    x = torch.randn((len(coords), 16), device="cuda", generator=g)
    w = torch.randn((27, 1, 16, 16), device="cuda", generator=g) * (2.0 / (16 * 27)) ** 0.5

    def build1():
        md = M.Metadata(3)
        md.inputLayer(s128, cd, x, 0, 0)
        return sync_ms(lambda: M._lib.check(L.scn_md_submanifold_rules(md._h, md._s(s128), md._s(three), stream))), md
    rb_ms = _host_timed(torch, build1)
    _, md = build1()
    _, macs = md.submanifoldConvolution(s128, three, x, w, None)
    R, n = macs / 256, len(coords)
    ms = _timed(torch, lambda: md.submanifoldConvolution(s128, three, x, w, None, want_macs=False))
    rows["config1"] = {"workload": "SubmanifoldConvolution 3^3 16->16, batch 2, 128^3, %d sites, %d rules" % (n, R),
                       "ms": round(ms, 4), "gflops": round(2 * macs / (ms * 1e-3) / 1e9, 1),
                       "sites_per_s": round(n / (ms * 1e-3)), "roofline": roofline_for(16, 16, R, n, 27, ms),
                       "rulebook_ms": round(rb_ms, 4),
                       "rulebook_roofline": hbm_roofline(subm_rulebook_bytes(n, 27, R), rb_ms)}
    del md

    # configuration 2: 2-D VGG (examples/hello-world.py:19-30), 100 samples of pen strokes in a 64x64
    # canvas; the three MaxPooling 3/2 need an input extent of 8k + 7: spatial size 71, output 100x32x8x8
    torch.manual_seed(2)
    model = scn.Sequential().add(scn.SparseVggNet(2, 1, [['C', 8], ['C', 8], ['MP', 3, 2], ['C', 16], ['C', 16],
                                                         ['MP', 3, 2], ['C', 24], ['C', 24], ['MP', 3, 2]])).add(
        scn.SubmanifoldConvolution(2, 24, 32, 3, False)).add(scn.BatchNormReLU(32)).add(
        scn.SparseToDense(2, 32)).cuda().eval()
    c2 = synthetic.strokes2d(seed=2000, batch=100, canvas=64, spatial=71)
    c2d = torch.as_tensor(c2).cuda()
    f2 = torch.ones((len(c2), 1), device="cuda")
    layer = scn.InputLayer(2, 71, mode=3)
    with torch.no_grad():
        def cold2():
            out = []
            ms = sync_ms(lambda: out.append(model(layer([c2d, f2]))))
            return ms, out
        cold_ms = _host_timed(torch, cold2, reps=6)
        xin = layer([c2d, f2])
        model(xin)
        warm_ms = float(np.median([sync_ms(lambda: model(xin)) for _ in range(7)]))
    rows["config2"] = {"workload": "2-D SparseVggNet C8,C8,MP3/2,C16,C16,MP3/2,C24,C24,MP3/2 + SubmanifoldConvolution "
                                   "24->32 + BatchNormReLU + SparseToDense, batch 100, spatial 71 (64x64 canvas), "
                                   "%d active sites" % len(c2),
                       "ms_per_batch": round(cold_ms, 3), "warm_ms_per_batch": round(warm_ms, 3),
                       "samples_per_s": round(100 / (cold_ms * 1e-3))}
    del xin

    # configuration 4 as a tree at 4094^3: h = Convolution 2^3/2 32->64; MaxPooling(3, 2)(h);
    # BatchNormReLU(Deconvolution 2^3/2 64->32 (h))
    coords = synthetic.room_scene(seed=4000, target=1000000, spatial=4094)
    cd = torch.as_tensor(coords).cuda()
    n = len(coords)
    sz = [torch.LongTensor([v] * 3) for v in (4094, 2047, 1023)]
    two, thr = torch.LongTensor([2] * 3), torch.LongTensor([3] * 3)
    x = torch.randn((n, 32), device="cuda", generator=g)
    w1 = torch.randn((8, 1, 32, 64), device="cuda", generator=g) * 0.1
    w2 = torch.randn((8, 1, 64, 32), device="cuda", generator=g) * 0.1
    bn = (torch.zeros(32, device="cuda"), torch.ones(32, device="cuda"), None, None, 1e-4, 0.0)

    def build4():
        md = M.Metadata(3)
        md.inputLayer(sz[0], cd, x, 0, 0)
        a = sync_ms(lambda: M._lib.check(L.scn_md_strided_rules(md._h, md._s(sz[0]), md._s(sz[1]), md._s(two),
                                                                  md._s(two), stream)))
        b = sync_ms(lambda: M._lib.check(L.scn_md_strided_rules(md._h, md._s(sz[1]), md._s(sz[2]), md._s(thr),
                                                                  md._s(two), stream)))
        return (a, b), md
    t = []
    for _ in range(5):
        ab, md = build4()
        t.append(ab)
        if len(t) < 5:
            del md
    rb1, rb2 = (float(np.median([v[i] for v in t[1:]])) for i in range(2))
    n1, n2 = md.getNActive(sz[1]), md.getNActive(sz[2])
    h, _ = md.convolution(sz[0], sz[1], two, two, x, w1, None)
    sizes = (C.c_int64 * 27)()
    M._lib.check(L.scn_rules_sizes(md._h, 1, md._s(sz[1]), md._s(sz[2]), md._s(thr), md._s(two), stream, sizes))
    R2 = int(sum(sizes))
    ms_conv = _timed(torch, lambda: md.convolution(sz[0], sz[1], two, two, x, w1, None, want_macs=False))
    ms_mp = _timed(torch, lambda: md.maxPooling(sz[1], sz[2], thr, two, h, 0))
    ms_dc = _timed(torch, lambda: md.deconvolution(sz[1], sz[0], two, two, h, w2, None, post=bn, want_macs=False))

    def tree():
        hh, _ = md.convolution(sz[0], sz[1], two, two, x, w1, None, want_macs=False)
        md.maxPooling(sz[1], sz[2], thr, two, hh, 0)
        md.deconvolution(sz[1], sz[0], two, two, hh, w2, None, post=bn, want_macs=False)
    ms_tree = _timed(torch, tree)
    rows["config4"] = {
        "workload": "strided tree on a %d-site room scene in 4094^3: Convolution 2^3/2 32->64 (-> %d sites), "
                    "MaxPooling(3, 2) (-> %d sites), Deconvolution 2^3/2 64->32 + BatchNormReLU(32)" % (n, n1, n2),
        "tree_ms": round(ms_tree, 4),
        "rulebook_2s2_ms": round(rb1, 4),
        "rulebook_2s2_roofline": hbm_roofline(strided_rulebook_bytes(n, n1, n), rb1),
        "rulebook_3s2_ms": round(rb2, 4),
        "rulebook_3s2_roofline": hbm_roofline(strided_rulebook_bytes(n1, n2, R2), rb2),
        "convolution_ms": round(ms_conv, 4),
        "convolution_roofline": hbm_roofline(conv_bytes(n, n1, 8, 32, 64), ms_conv),
        "maxpooling_3s2_ms": round(ms_mp, 4),
        "maxpooling_3s2_roofline": hbm_roofline(R2 * 64 * 4 + 8 * R2 + n2 * 64 * 4, ms_mp),
        "deconvolution_bn_ms": round(ms_dc, 4),
        "deconvolution_bn_roofline": hbm_roofline(conv_bytes(n, n, 8, 64, 32), ms_dc)}
    return rows


def other_ops(sites, seed, backward=True):
    """The rest of the path on the same kind of scene, each op by itself with inputs resident
    in HBM: ms per call (median of 5 timings of 8 calls back to back, HIP events on the launch
    stream) and the algorithmic bytes it has to move, against the 8 TB/s of HBM.  Rulebook builds are timed from the host (they
    synchronise)."""
    import torch
    import sparseconvnet_amd as scn
    from sparseconvnet_amd import metadata as M
    from sparseconvnet_amd import synthetic

    def timed(fn, reps=5, inner=8):
        # `inner` calls back to back between one pair of events: these ops last 25-100 us, and a
        # single call between two events measures the launch as much as the kernel
        fn()
        ms = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(inner):
                fn()
            e1.record()
            torch.cuda.synchronize()
            ms.append(e0.elapsed_time(e1) / inner)
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
    # int64 coordinates and features of every point read, the sites' features written
    out.append(row("InputLayer mode 4: rules + level + forward, 3 planes (%d points -> %d sites)" % (npts, n), ms,
                   npts * 4 * 8 + npts * 3 * 4 + n * 3 * 4, points_per_s=round(npts / (ms * 1e-3))))
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
    out.append(row("BatchNormReLU eval (stand-alone pass), 64 planes", ms, 2 * n * 64 * 4 + 16 * 64))

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
    out.append(row("strided rulebook 2^3 / stride 2 + output level (%d -> %d sites)" % (n, nc), ms,
                   strided_rulebook_bytes(n, nc, n), sites_per_s=round(n / (ms * 1e-3))))
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

    if backward:
        # gradients of the same operators on the same scene (bytes: every array each reads or writes, once)
        d64, d32 = torch.randn_like(x64), torch.randn_like(x32)
        dc64, dc32 = torch.randn_like(yc), torch.randn_like(xc32)
        mp = md.maxPooling(sz, half, two, two, x32, 0)
        rm, rv = torch.zeros(64, device="cuda"), torch.ones(64, device="cuda")
        gam, bet = torch.ones(64, device="cuda"), torch.zeros(64, device="cuda")
        ms = timed(lambda: md.batchNormTrain(x64, rm, rv, gam, bet, 1e-4, 0.9, 0.0))
        out.append(row("BatchNormReLU training forward, 64 planes", ms, 3 * n * 64 * 4))
        y_bn, sm, si = md.batchNormTrain(x64, rm, rv, gam, bet, 1e-4, 0.9, 0.0)
        ms = timed(lambda: md.batchNormBackward(x64, y_bn, d64, sm, si, gam, 0.0, True))
        out.append(row("BatchNormReLU backward, 64 planes", ms, 7 * n * 64 * 4))
        ms = timed(lambda: md.convolutionBackward(sz, half, two, two, x32, dc64, w_dn, False))
        out.append(row("Convolution 2^3 / stride 2 backward, 32 -> 64", ms, 2 * (n * 32 * 4 + nc * 64 * 4) + 16 * n,
                       gflops=round(4.0 * n * 32 * 64 / (ms * 1e-3) / 1e9, 1)))
        ms = timed(lambda: md.deconvolutionBackward(half, sz, two, two, yc, d32, w_up, False))
        out.append(row("Deconvolution 2^3 / stride 2 backward, 64 -> 32", ms, 2 * (nc * 64 * 4 + n * 32 * 4) + 16 * n,
                       gflops=round(4.0 * n * 64 * 32 / (ms * 1e-3) / 1e9, 1)))
        ms = timed(lambda: md.networkInNetworkBackward(x64, d32, w_nin, False))
        out.append(row("NetworkInNetwork backward, 64 -> 32", ms, 2 * n * 64 * 4 + 2 * n * 32 * 4,
                       gflops=round(4.0 * n * 64 * 32 / (ms * 1e-3) / 1e9, 1)))
        ms = timed(lambda: md.maxPoolingBackward(sz, half, two, two, x32, mp, dc32, 0))
        out.append(row("MaxPooling 2^3 / stride 2 backward, 32 planes", ms, 2 * n * 32 * 4 + 8 * n + 2 * nc * 32 * 4))
        ms = timed(lambda: md.averagePoolingBackward(sz, half, two, two, x32.shape, dc32, 0))
        out.append(row("AveragePooling 2^3 / stride 2 backward, 32 planes", ms, n * 32 * 4 + 8 * n + nc * 32 * 4))
        ms = timed(lambda: md.unPoolingBackward(half, sz, two, two, xc32.shape, d32, 0))
        out.append(row("UnPooling 2^3 / stride 2 backward, 32 planes", ms, nc * 32 * 4 + 8 * n + n * 32 * 4))
        ms = timed(lambda: md.inputLayerBackward(x3))
        out.append(row("InputLayer backward, 3 planes", ms, npts * 12 + npts * 4 + n * 12))
        dpts = torch.randn((npts, 32), device="cuda", generator=g)
        ms = timed(lambda: md.outputLayerBackward(dpts, n))
        out.append(row("OutputLayer backward, 32 planes", ms, npts * 32 * 4 + npts * 4 + n * 32 * 4 + n * 8))
        ms = timed(lambda: md.activePoolingBackward(half, yc.shape, torch.randn((1, 64), device="cuda"), True))
        out.append(row("ActivePooling backward, 64 planes, %d sites" % nc, ms, nc * 64 * 4))
        del d64, d32, dc64, dc32, mp, y_bn, dpts

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
        if len(t) < 4:
            del m3
    ms = float(np.median(t[1:]))
    total = sum(levels)
    # every level's submanifold rulebook and the strided one to the next level, by the same formulas
    byts = 0.0
    cnt = (C.c_int64 * 27)()
    for l, nl in enumerate(levels):
        if not nl:
            continue
        M._lib.check(L.scn_rules_sizes(m3._h, 0, m3._s([4096 >> l] * 3), m3._s(3), None, None, stream, cnt))
        byts += subm_rulebook_bytes(nl, 27, sum(cnt))
        if l + 1 < len(levels):
            byts += strided_rulebook_bytes(nl, levels[l + 1], nl)
    del m3
    out.append(row("precompute_metadata(2): 3^3 and 2^3/stride-2 rulebooks of all %d levels (%d sites in all)"
                   % (sum(1 for v in levels if v), total), ms, byts, sites_per_s=round(total / (ms * 1e-3))))
    # per-sample mean of the active rows (one sample here: a column mean over every row), on the
    # level a stride-2 convolution made (rows in site order) and on the input level (rows in the
    # caller's point order: the sums walk the samples' site ranges, a gather there)
    ms = timed(lambda: md.activePooling(half, yc, True))
    out.append(row("ActivePooling (mean), 64 planes, %d sites (level of a stride-2 convolution)" % yc.shape[0], ms,
                   yc.shape[0] * 64 * 4 + 64 * 4))
    ms = timed(lambda: md.activePooling(sz, x32, True))
    out.append(row("ActivePooling (mean), 32 planes, input level", ms, n * 32 * 4 + 32 * 4))
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
    ap.add_argument("--cpu-port-sites", type=int, default=60000)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-configs", action="store_true")
    ap.add_argument("--pairs", default="")
    ap.add_argument("--no-unet", action="store_true")
    ap.add_argument("--no-ops", action="store_true")
    ap.add_argument("--no-bf16", action="store_true")
    ap.add_argument("--no-backward", action="store_true")
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
    # every pair once more on its own, back to back: a short launch right behind the long 256->256 one of
    # the step above runs slower than among launches of its own kind
    alone_ms = []
    for wk in work:
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        conv(*wk)
        a.record()
        for _ in range(args.steps):
            conv(*wk)
        b.record()
        torch.cuda.synchronize()
        alone_ms.append(a.elapsed_time(b) / args.steps)
    total_flops = sum(2.0 * R * cin * cout for cin, cout in pairs)
    value = total_flops / (ms_per_step * 1e-3) / 1e9

    default_workload = args.sites == 1000000 and args.seed == 3000 and args.order == "shuffled"
    traffic = measured_traffic() if default_workload else {}
    sweep = []
    for (cin, cout), ms, alone in zip(pairs, per_pair_ms, alone_ms):
        sweep.append({"nIn": cin, "nOut": cout, "ms": round(ms, 4), "ms_back_to_back": round(alone, 4),
                      "gflops": round(2.0 * R * cin * cout / (ms * 1e-3) / 1e9, 1),
                      "sites_per_s": round(n / (ms * 1e-3)),
                      "roofline": roofline_for(cin, cout, R, n, 27, ms, traffic.get((cin, cout)))})
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
        "rulebook_roofline": hbm_roofline(subm_rulebook_bytes(n, 27, R), rulebook_ms),
        "roofline": roof, "sweep": sweep,
    }
    if not args.no_backward:
        # Backward pass of the same layers on the same scene (gradients of input rows, weights and
        # bias): R.nIn.nOut multiply-adds for the input gradient and as many for the weight
        # gradient, twice the forward pass's count.
        bw = []
        for cin, cout, x, w, y in work:
            if cin * cout > 128 * 128:
                continue  # the widest layer: nothing the narrower ones do not show, 25 ms per call
            d_y = torch.randn((n, cout), device="cuda", generator=g)
            d_x, d_w, d_b = torch.empty_like(x), torch.empty_like(w), torch.empty(cout, device="cuda")

            def bwd():
                _lib.check(L.scn_subm_conv_bwd(h, sp, fs, C.c_void_p(x.data_ptr()), C.c_void_p(d_x.data_ptr()),
                                               C.c_void_p(d_y.data_ptr()), C.c_void_p(w.data_ptr()),
                                               C.c_void_p(d_w.data_ptr()), C.c_void_p(d_b.data_ptr()), cin, cout, 1, stream))
            ms = _timed(torch, bwd, reps=3)
            bw.append({"nIn": cin, "nOut": cout, "ms": round(ms, 4),
                       "gflops": round(4.0 * R * cin * cout / (ms * 1e-3) / 1e9, 1),
                       "frac_mfma_fp32": round(4.0 * R * cin * cout / (ms * 1e-3) / 1e12 / MFMA_FP32_TFLOPS, 4)})
            del d_y, d_x, d_w, d_b
        out["sweep_backward"] = bw
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
                       "speedup_vs_f32": round(per_pair_ms[i] / ms, 2),
                       "roofline": roofline_bf16(wk[0], wk[1], R, n, 27, ms)})
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
    if not args.no_configs:
        out["configs"] = config_rows()
    if not args.no_ops:
        out["other_ops"] = other_ops(args.unet_sites, 5000, backward=not args.no_backward)
    if not args.no_unet:
        out["unet"] = unet_scene(args.unet_sites, 5000)
        if not args.no_residual:
            out["unet"].update(unet_scene(args.unet_sites, 5000, residual=True))
            out["unet"].update(unet_scene(args.unet_sites, 7000, reps=2, batch=4))
        if not args.no_backward:
            out["unet"].update(unet_train_step(args.unet_sites, 5000))
        if not args.no_bf16:
            import sparseconvnet_amd as scn
            scn.bf16_mfma = True
            u = unet_scene(args.unet_sites, 5000)
            scn.bf16_mfma = False
            out["unet"].update({"unet_bf16_ms_per_scene": u["unet_ms_per_scene"], "unet_bf16_warm_ms": u["unet_warm_ms"]})
    if not args.no_cpu:
        # the reference's own CPU sources where oracle/_ref was built, else this repository's port;
        # the port is listed as well (naive inner loops: a smaller scene keeps it bounded)
        ref = cpu_baseline("reference", args.cpu_sites, args.seed, compare=gpu_outputs)
        port = cpu_baseline("port", args.cpu_port_sites, args.seed, compare=gpu_outputs)
        out["cpu_baseline"] = ref if ref is not None else port
        if ref is not None and port is not None:
            out["cpu_baseline_port"] = port
    print(json.dumps(out))


if __name__ == "__main__":
    main()
