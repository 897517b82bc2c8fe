"""Whole networks through the module API on the GPU against the CPU oracle run over the same
module tree and parameters (tests/oracle_model.py).  fp32 tolerance 1e-4 rel / 1e-5 abs."""
import numpy as np
import pytest
import torch

import checks
import oracle_model
import sparseconvnet_amd as scn
from oracle import cpu_path
from sparseconvnet_amd import synthetic
from test_modules_api import hello_world_model

pytestmark = pytest.mark.gpu


def randomise_bn(model, seed):
    g = torch.Generator().manual_seed(seed)
    for m in model.modules():
        if isinstance(m, scn.BatchNormalization):
            m.running_mean.copy_(torch.randn(m.nPlanes, generator=g))
            m.running_var.copy_(torch.rand(m.nPlanes, generator=g) + 0.5)


def test_hello_world_shape():
    # examples/hello-world.py: the output of the two-sample message batch is 2x32x10x10
    torch.manual_seed(0)
    model = hello_world_model().cuda().eval()
    size = model.input_spatial_size(torch.LongTensor([10, 10]))
    msgs = [[" X   X  XXX  X    X    XX     X       X   XX   XXX   X    XXX   ",
             " X   X  X    X    X   X  X    X       X  X  X  X  X  X    X  X  ",
             " XXXXX  XX   X    X   X  X    X   X   X  X  X  XXX   X    X   X ",
             " X   X  X    X    X   X  X     X X X X   X  X  X  X  X    X  X  ",
             " X   X  XXX  XXX  XXX  XX       X   X     XX   X  X  XXX  XXX   "],
            [" XXX              XXXXX      x   x     x  xxxxx  xxx ",
             " X  X  X   XXX       X       x   x x   x  x     x  x ",
             " XXX                X        x   xxxx  x  xxxx   xxx ",
             " X     X   XXX       X       x     x   x      x    x ",
             " X     X          XXXX   x   x     x   x  xxxx     x "]]
    loc, feat = [], []
    for b, msg in enumerate(msgs):
        for y, line in enumerate(msg):
            for x, c in enumerate(line):
                if c == 'X':
                    loc.append([y, x, b])
                    feat.append([1.0])
    inp = scn.InputLayer(2, size)([torch.LongTensor(loc), torch.FloatTensor(feat).cuda()])
    assert inp.batch_size() == 2 and inp.features.shape == (len(loc), 1)
    assert (inp.get_spatial_locations() == torch.LongTensor(loc)).all()
    with torch.no_grad():
        out = model(inp)
    assert tuple(out.shape) == (2, 32, 10, 10) and out.is_cuda
    assert torch.isfinite(out).all() and (out >= 0).all() and out.abs().sum() > 0
    # "Alternatively" (examples/hello-world.py:72-92): the same batch through BLInputLayer
    batch = []
    for b in range(2):
        sel = [i for i, l in enumerate(loc) if l[2] == b]
        batch.append([torch.LongTensor([loc[i][:2] for i in sel]), torch.FloatTensor([feat[i] for i in sel])])
    batch = scn.prepare_BLInput(batch)
    assert tuple(batch[0].shape) == (2, max(sum(l[2] == b for l in loc) for b in range(2)), 2)
    batch[1] = batch[1].cuda()
    with torch.no_grad():
        out_bl = model(scn.BLInputLayer(2, size)(batch))
    assert torch.allclose(out_bl, out, rtol=1e-4, atol=1e-5)


def _run_both(model, inp_layer, x):
    p = cpu_path.CpuPath(inp_layer.dimension, "oracle")
    t = oracle_model.run(inp_layer, p, x)
    want = oracle_model.run(model, p, t)
    with torch.no_grad():
        got = model.cuda()(inp_layer([x[0], x[1].cuda()]))
    return got, want, p


def test_unet_vs_oracle(oracle_built):
    """Configuration 5 at reduced width and size: InputLayer mode 4 (duplicates averaged),
    SubmanifoldConvolution 3->8, UNet(reps=2, 4 levels), OutputLayer, Linear."""
    torch.manual_seed(5)
    m = 8
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 2, [m, 2 * m, 3 * m, 4 * m], False)).add(scn.OutputLayer(3)).eval()
    randomise_bn(model, 5)
    linear = torch.nn.Linear(m, 20)
    coords = synthetic.scene_batch(seed=5000, batch=2, target=6000, spatial=64, n_boxes=8,
                                   duplicate_fraction=0.3)
    rng = np.random.default_rng(5)
    feats = rng.uniform(-1, 1, size=(len(coords), 3)).astype(np.float32)
    inp_layer = scn.InputLayer(3, 64, mode=4)
    x = [torch.as_tensor(coords), torch.as_tensor(feats)]
    got, want, p = _run_both(model, inp_layer, x)
    assert got.shape == (len(coords), m)
    checks.assert_close(got.cpu().numpy(), want, "U-Net output rows")
    with torch.no_grad():
        logits = linear.cuda()(got)
    assert logits.shape == (len(coords), 20)


@pytest.mark.parametrize("batch,target,seed", [(1, 120000, 5100), (2, 40000, 5101)])
def test_unet_full_width_vs_oracle(oracle_built, batch, target, seed):
    """Configuration 5 at its full width (examples/ScanNet/unet.py:25-38): m = 32, 7 levels with
    32 ... 224 planes (joins up to 448), two blocks per level, InputLayer mode 4 with 30 %
    repeated points, in a 4096^3 grid; only the scene is smaller than the benchmark's (levels of
    120 k, 29 k, 7 k, ... sites, which takes every convolution kernel family and the small-level
    paths).  GPU against the oracle over the same module tree, 1e-4 relative / 1e-5 absolute."""
    torch.manual_seed(seed)
    m = 32
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 2, [m * (i + 1) for i in range(7)], False)).add(scn.OutputLayer(3)).eval()
    randomise_bn(model, seed)
    if batch == 1:
        coords = synthetic.room_scene(seed=seed, target=target, spatial=4096, duplicate_fraction=0.3)
    else:
        coords = synthetic.scene_batch(seed=seed, batch=batch, target=target, spatial=4096, duplicate_fraction=0.3)
    rng = np.random.default_rng(seed)
    feats = rng.uniform(-1, 1, size=(len(coords), 3)).astype(np.float32)
    inp_layer = scn.InputLayer(3, 4096, mode=4)
    got, want, p = _run_both(model, inp_layer, [torch.as_tensor(coords), torch.as_tensor(feats)])
    assert got.shape == (len(coords), m)
    assert len(p.spatial_locations(64)) > 0  # all seven levels are populated
    checks.assert_close(got.cpu().numpy(), want, "full-width U-Net output rows (batch %d)" % batch)


def test_residual_unet_vs_oracle(oracle_built):
    """The ScanNet example's residual variant at reduced width: blocks of two BN + convolution
    pairs added to the block input, through a NetworkInNetwork where the plane count changes."""
    torch.manual_seed(6)
    m = 8
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 2, [m, 2 * m, 3 * m, 4 * m], True)).add(scn.BatchNormReLU(m)).add(scn.OutputLayer(3)).eval()
    randomise_bn(model, 6)
    coords = synthetic.scene_batch(seed=5001, batch=2, target=6000, spatial=64, n_boxes=8,
                                   duplicate_fraction=0.3)
    rng = np.random.default_rng(6)
    feats = rng.uniform(-1, 1, size=(len(coords), 3)).astype(np.float32)
    inp_layer = scn.InputLayer(3, 64, mode=4)
    got, want, p = _run_both(model, inp_layer, [torch.as_tensor(coords), torch.as_tensor(feats)])
    assert got.shape == (len(coords), m)
    checks.assert_close(got.cpu().numpy(), want, "residual U-Net output rows")


def test_average_and_unpooling_modules_vs_oracle(oracle_built):
    """AveragePooling down and UnPooling back up around a convolution, joined with the skip
    path (the shape of FullyConvolutionalNet's levels, networkArchitectures.py:259-312)."""
    torch.manual_seed(7)
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, 8, 3, False)).add(scn.BatchNormReLU(8)).add(
        scn.ConcatTable().add(scn.Identity()).add(
            scn.Sequential().add(scn.AveragePooling(3, 2, 2)).add(scn.SubmanifoldConvolution(3, 8, 12, 3, True))
            .add(scn.BatchNormLeakyReLU(12)).add(scn.UnPooling(3, 2, 2)))).add(scn.JoinTable()).add(
        scn.AveragePooling(3, 2, 2, nFeaturesToDrop=4)).eval()
    randomise_bn(model, 7)
    assert (model.input_spatial_size(torch.LongTensor([15] * 3)) == 30).all()
    coords = synthetic.scene_batch(seed=7000, batch=3, target=3000, spatial=30, n_boxes=5)
    rng = np.random.default_rng(7)
    feats = rng.uniform(-1, 1, size=(len(coords), 3)).astype(np.float32)
    inp_layer = scn.InputLayer(3, 30, mode=3)
    got, want, p = _run_both(model, inp_layer, [torch.as_tensor(coords), torch.as_tensor(feats)])
    assert got.features.shape == (p.nactive(15), 16) and (got.spatial_size == 15).all()
    rows = lambda loc: cpu_path.canon_rows(loc)  # noqa: E731
    checks.assert_close(got.features.cpu().numpy()[rows(got.get_spatial_locations().numpy())],
                        want.features[rows(p.spatial_locations(15))], "pooling network")


def test_bl_layers_network_vs_oracle(oracle_built):
    """BLInputLayer (mode 4, with empty positions) -> convolutions -> BLOutputLayer."""
    torch.manual_seed(8)
    model = scn.Sequential().add(scn.SubmanifoldConvolution(2, 4, 8, 3, True)).add(scn.BatchNormReLU(8)).add(
        scn.SubmanifoldConvolution(2, 8, 6, 3, False)).add(scn.BLOutputLayer(2)).eval()
    randomise_bn(model, 8)
    rng = np.random.default_rng(8)
    coords = rng.integers(0, 24, (5, 200, 2)).astype(np.int64)
    coords[rng.random((5, 200)) < 0.15] = -1
    feats = rng.normal(size=(5, 200, 4)).astype(np.float32)
    inp_layer = scn.BLInputLayer(2, 24, mode=4)
    got, want, p = _run_both(model, inp_layer, [torch.as_tensor(coords), torch.as_tensor(feats)])
    assert tuple(got.shape) == (5, 200, 6)
    checks.assert_close(got.cpu().numpy(), want, "batch-by-length network")
    assert (got.cpu().numpy()[coords[:, :, 0] < 0] == 0).all()


def test_vgg2d_vs_oracle(oracle_built):
    torch.manual_seed(2)
    model = hello_world_model().eval()
    randomise_bn(model, 2)
    coords = synthetic.strokes2d(seed=2000, batch=100, canvas=64, spatial=71)
    feats = np.ones((len(coords), 1), np.float32)
    inp_layer = scn.InputLayer(2, 71, mode=3)
    got, want, _ = _run_both(model, inp_layer, [torch.as_tensor(coords), torch.as_tensor(feats)])
    assert tuple(got.shape) == (100, 32, 8, 8)
    checks.assert_close(got.cpu().numpy(), want, "2-D VGG dense output")


def test_eval_mode_batch_norm_refuses_backward():
    """batchNormalization.py:147 asserts ctx.train in backward; so does this build, also when the
    eval-mode batch norm was applied inside a convolution."""
    bn = scn.BatchNormReLU(4).cuda().eval()
    feats = torch.ones(3, 4).cuda().requires_grad_()
    t = scn.InputLayer(2, 8)([torch.LongTensor([[1, 1, 0], [2, 2, 0], [5, 5, 0]]), feats])
    with pytest.raises(AssertionError):
        bn(t).features.sum().backward()
    model = scn.Sequential().add(scn.SubmanifoldConvolution(2, 4, 4, 3, False)).add(scn.BatchNormReLU(4)).cuda().eval()
    with pytest.raises(AssertionError):
        model(t).features.sum().backward()


def test_module_chain_gradients_vs_oracle(oracle_built):
    """A chain of every differentiable module in training mode (InputLayer mode 4, submanifold
    convolution with bias, BatchNormReLU, strided convolution, BatchNormLeakyReLU, max and average
    pooling side branches, transposed convolution, NetworkInNetwork, OutputLayer): the gradients
    torch.autograd collects through this build's Functions against the same chain walked backwards
    by hand with the oracle's backward calls."""
    torch.manual_seed(31)
    rng = np.random.default_rng(31)
    coords = synthetic.room_scene(seed=3100, target=3000, spatial=30, duplicate_fraction=0.3)
    feats = rng.normal(size=(len(coords), 3)).astype(np.float32)
    conv1 = scn.SubmanifoldConvolution(3, 3, 8, 3, True).cuda()
    bn1 = scn.BatchNormReLU(8).cuda()
    down = scn.Convolution(3, 8, 12, 2, 2, False).cuda()
    bn2 = scn.BatchNormLeakyReLU(12, leakiness=0.2).cuda()
    up = scn.Deconvolution(3, 12, 8, 2, 2, True).cuda()
    nin = scn.NetworkInNetwork(8, 5, True).cuda()
    mp, ap, unp = scn.MaxPooling(3, 2, 2).cuda(), scn.AveragePooling(3, 2, 2).cuda(), scn.UnPooling(3, 2, 2).cuda()
    with torch.no_grad():
        conv1.bias.normal_()
        up.bias.normal_()
        nin.bias.normal_()
        for b in (bn1, bn2):
            b.weight.uniform_(0.5, 1.5)
            b.bias.normal_()
    mods = [conv1, bn1, down, bn2, up, nin]
    for m in mods:
        m.train()
    f = torch.as_tensor(feats).cuda().requires_grad_()
    x0 = scn.InputLayer(3, 30, mode=4)([torch.as_tensor(coords), f])
    h1 = bn1(conv1(x0))
    h2 = bn2(down(h1))
    pooled = scn.AddTable()([mp(h1), ap(h1), scn.Identity()(mp(h1))])  # max pooling counted twice
    side = unp(pooled)
    y = nin(scn.AddTable()([up(h2), side]))
    out = scn.OutputLayer(3)(y)
    g_out = torch.as_tensor(rng.normal(size=tuple(out.shape)).astype(np.float32)).cuda()
    (out * g_out).sum().backward()

    # the same chain on the oracle, forwards and then backwards by hand
    o = cpu_path.CpuPath(3, "oracle")
    P = lambda t: t.detach().cpu().numpy()
    o.input_layer(30, coords, 0, 4)
    a0 = o.input_fwd(feats)
    a1, _ = o.subm_conv(30, 3, a0, P(conv1.weight), P(conv1.bias))
    b1, sm1, si1, _, _ = o.bn_train(a1, np.zeros(8), np.ones(8), P(bn1.weight), P(bn1.bias), 1e-4, 0.99, 0.0)
    a2, _ = o.conv(30, 15, 2, 2, b1, P(down.weight))
    b2, sm2, si2, _, _ = o.bn_train(a2, np.zeros(12), np.ones(12), P(bn2.weight), P(bn2.bias), 1e-4, 0.99, 0.2)
    m1, v1 = o.maxpool(30, 15, 2, 2, b1), o.avgpool(30, 15, 2, 2, b1)
    pooled_o = m1 + v1 + m1
    side_o = o.unpool(15, 30, 2, 2, pooled_o)
    a3, _ = o.deconv(15, 30, 2, 2, b2, P(up.weight), P(up.bias))
    s3 = a3 + side_o
    yo, _ = o.nin(s3, P(nin.weight), P(nin.bias))
    checks.assert_close(P(out), o.output_fwd(yo), "forward of the chain")
    d_y = o.output_bwd(P(g_out))
    d_s3, d_wn, d_bn = o.nin_bwd(s3, d_y, P(nin.weight), True)
    d_b2, d_wu, d_bu = o.deconv_bwd(15, 30, 2, 2, b2, d_s3, P(up.weight), True)
    d_pooled = o.unpool_bwd(15, 30, 2, 2, 8, d_s3)
    d_b1 = 2 * o.maxpool_bwd(30, 15, 2, 2, b1, m1, d_pooled) + o.avgpool_bwd(30, 15, 2, 2, 8, d_pooled)
    d_a2, d_g2, d_be2 = o.bn_bwd(a2, b2, d_b2, sm2, si2, P(bn2.weight), 0.2)
    d_b1c, d_wd, _ = o.conv_bwd(30, 15, 2, 2, b1, d_a2, P(down.weight))
    d_b1 = d_b1 + d_b1c
    d_a1, d_g1, d_be1 = o.bn_bwd(a1, b1, d_b1, sm1, si1, P(bn1.weight), 0.0)
    d_a0, d_w1, d_bias1 = o.subm_conv_bwd(30, 3, a0, d_a1, P(conv1.weight), True)
    d_f = o.input_bwd(d_a0)
    # (the gradients compared below do not depend on how either side numbers the coarse rows)
    for got, want, what in ((f.grad, d_f, "input features"), (conv1.weight.grad, d_w1, "conv1 weight"),
                            (bn1.weight.grad, d_g1, "bn1 weight"),
                            (bn1.bias.grad, d_be1, "bn1 bias"), (down.weight.grad, d_wd, "strided weight"),
                            (bn2.weight.grad, d_g2, "bn2 weight"), (bn2.bias.grad, d_be2, "bn2 bias"),
                            (up.weight.grad, d_wu, "transposed weight"), (up.bias.grad, d_bu, "transposed bias"),
                            (nin.weight.grad, d_wn, "nin weight"), (nin.bias.grad, d_bn, "nin bias")):
        checks.assert_close(P(got), want, "gradient of " + what)
    # a bias in front of a training-mode batch norm has gradient zero: both sides hold the rounding
    # noise of a column sum that cancels, so the bound is relative to the summands
    assert (np.abs(P(conv1.bias.grad) - d_bias1) <= 1e-6 * np.abs(d_a1).sum(0)).all()
    assert (np.abs(d_bias1) <= 1e-6 * np.abs(d_a1).sum(0)).all()
    # running statistics moved towards the batch's (momentum 0.99 weights the old value)
    checks.assert_close(P(bn1.running_mean), 0.01 * a1.astype(np.float64).mean(0), "running mean")


def test_unet_trains():
    """A small U-Net (residual blocks, training-mode batch norms, JoinTable / AddTable through
    torch) fits a toy per-point regression target: gradients reach every parameter and the loss
    falls under plain SGD."""
    torch.manual_seed(32)
    m = 8
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 1, [m, 2 * m, 3 * m], True)).add(scn.BatchNormReLU(m)).add(scn.OutputLayer(3)).cuda().train()
    head = torch.nn.Linear(m, 1).cuda()
    coords = synthetic.room_scene(seed=3200, target=4000, spatial=64, duplicate_fraction=0.2)
    feats = torch.rand((len(coords), 3), device="cuda")
    target = (torch.as_tensor(coords[:, 2:3]).float().cuda() / 64.0)
    params = list(model.parameters()) + list(head.parameters())
    opt = torch.optim.SGD(params, lr=0.05, momentum=0.9)
    layer = scn.InputLayer(3, 64, mode=4)
    losses = []
    for step in range(12):
        opt.zero_grad()
        pred = head(model(layer([torch.as_tensor(coords), feats])))
        loss = ((pred - target) ** 2).mean()
        loss.backward()
        if step == 0:
            assert all(p.grad is not None and torch.isfinite(p.grad).all() and p.grad.abs().sum() > 0 for p in params)
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < 0.5 * losses[0], losses


def test_empty_input_passes_through():
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, 4, 3, False)).add(scn.BatchNormReLU(4)).cuda().eval()
    t = scn.InputLayer(3, 16, mode=4)([torch.zeros((0, 4), dtype=torch.int64), torch.zeros((0, 3)).cuda()])
    with torch.no_grad():
        out = model(t)
    assert out.features.shape == (0, 4)


def test_fused_and_unfused_sequential_agree():
    """Sequential hands a batch normalisation in front of a convolution to that convolution;
    with sparseconvnet_amd.fuse_batchnorm off every module runs by itself.  Same result."""
    torch.manual_seed(7)
    m = 16
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 2, [m, 2 * m, 3 * m], False, leakiness=0.2)).add(scn.BatchNormReLU(m)).add(
        scn.OutputLayer(3)).cuda().eval()
    randomise_bn(model, 7)
    coords = synthetic.scene_batch(seed=7000, batch=2, target=8000, spatial=64, n_boxes=8)
    feats = torch.rand(len(coords), 3).cuda()
    inp_layer = scn.InputLayer(3, 64, mode=4)
    outs = []
    for fuse in (True, False):
        scn.fuse_batchnorm = fuse
        try:
            with torch.no_grad():
                outs.append(model(inp_layer([torch.as_tensor(coords), feats])).cpu().numpy())
        finally:
            scn.fuse_batchnorm = True
    checks.assert_close(outs[0], outs[1], "fused vs unfused")


def test_multiply_add_counter_matches_oracle(oracle_built):
    """forward_pass_multiplyAdd_count (sparseconvnet/__init__.py:7) is collected lazily from
    the library; it must equal the sum of the counts the reference returns per layer
    (CPU/Convolution.cpp:141), also when read twice, after a reset, and when the Metadata has
    already been dropped."""
    torch.manual_seed(11)
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, 8, 3, False)).add(
        scn.Convolution(3, 8, 16, 2, 2, False)).add(scn.SubmanifoldConvolution(3, 16, 16, 3, True)).add(
        scn.Deconvolution(3, 16, 8, 2, 2, False)).cuda().eval()
    coords = synthetic.scene_batch(seed=1100, batch=2, target=3000, spatial=32, n_boxes=5)
    feats = np.random.default_rng(11).normal(size=(len(coords), 3)).astype(np.float32)
    p = cpu_path.CpuPath(3, "oracle")
    p.input_layer(32, coords, 0, 4)
    x = p.input_fwd(feats)
    want = 0.0
    h, m1 = p.subm_conv(32, 3, x, np.zeros((27, 1, 3, 8), np.float32))
    p.strided_rules(32, 16, 2, 2)
    h, m2 = p.conv(32, 16, 2, 2, h, np.zeros((8, 1, 8, 16), np.float32))
    h, m3 = p.subm_conv(16, 3, h, np.zeros((27, 1, 16, 16), np.float32))
    h, m4 = p.deconv(16, 32, 2, 2, h, np.zeros((8, 1, 16, 8), np.float32))
    want = m1 + m2 + m3 + m4
    scn.forward_pass_multiplyAdd_count = 0
    scn.forward_pass_hidden_states = 0
    inp = scn.InputLayer(3, 32, mode=4)([torch.as_tensor(coords), torch.as_tensor(feats).cuda()])
    with torch.no_grad():
        out = model(inp)
    assert scn.forward_pass_multiplyAdd_count == want
    assert scn.forward_pass_multiplyAdd_count == want  # reading does not consume it
    with torch.no_grad():
        model(inp)  # rulebooks cached: the counts are known without a round trip
    assert scn.forward_pass_multiplyAdd_count == 2 * want
    scn.forward_pass_multiplyAdd_count = 0
    with torch.no_grad():
        out = model(scn.InputLayer(3, 32, mode=4)([torch.as_tensor(coords), torch.as_tensor(feats).cuda()]))
    del out, inp
    import gc
    gc.collect()
    assert scn.forward_pass_multiplyAdd_count == want
    assert scn.forward_pass_hidden_states > 0


def test_unet_scene_scale_invariants():
    """The ScanNet-style U-Net (m = 32, 7 levels, mode-4 input with duplicated points) on a
    250,000-point scene, where the oracle is too slow: the result does not depend on the order
    of the input points (rows follow their points), is bit-identical between a cold pass and a
    pass over cached rulebooks, and the fused and unfused batch norms agree."""
    torch.manual_seed(21)
    m = 32
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 2, [m, 2 * m, 3 * m, 4 * m, 5 * m, 6 * m, 7 * m], False)).add(scn.BatchNormReLU(m)).add(
        scn.OutputLayer(3)).cuda().eval()
    randomise_bn(model, 21)
    coords = synthetic.room_scene(seed=2100, target=200000, spatial=4096, duplicate_fraction=0.3)
    rng = np.random.default_rng(21)
    feats = rng.uniform(-1, 1, size=(len(coords), 3)).astype(np.float32)
    layer = scn.InputLayer(3, 4096, mode=4)

    def run(c, f, twice=False):
        with torch.no_grad():
            x = layer([torch.as_tensor(c).cuda(), torch.as_tensor(f).cuda()])
            y = model(x)
            if twice:
                return y.cpu().numpy(), model(x).cpu().numpy()
            return y.cpu().numpy()
    cold, warm = run(coords, feats, twice=True)
    assert cold.shape == (len(coords), m) and np.isfinite(cold).all() and np.abs(cold).max() > 0
    assert (cold == warm).all()
    perm = rng.permutation(len(coords))
    shuffled = run(coords[perm], feats[perm])
    # summation orders inside duplicate groups and pattern-sorted tiles may differ: tolerance, not bits
    checks.assert_close(shuffled, cold[perm], "permuted input points")
    scn.fuse_batchnorm = False
    try:
        unfused = run(coords, feats)
    finally:
        scn.fuse_batchnorm = True
    checks.assert_close(cold, unfused, "fused vs unfused U-Net")


def test_warm_forward_can_be_captured_in_a_graph():
    """With its rulebooks built, a forward pass enqueues kernels only (no host round trip, no
    memset nodes): captured once in a HIP graph, every replay reproduces the eager result, also
    with eager work between the replays."""
    torch.manual_seed(9)
    m = 16
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 1, [m, 2 * m, 3 * m], False)).add(scn.BatchNormReLU(m)).add(scn.OutputLayer(3)).cuda().eval()
    randomise_bn(model, 9)
    coords = synthetic.room_scene(seed=9000, target=20000, spatial=256, duplicate_fraction=0.2)
    feats = torch.rand((len(coords), 3), device="cuda")
    with torch.no_grad():
        x = scn.InputLayer(3, 256, mode=4)([torch.as_tensor(coords), feats])
        want = model(x)                      # builds every rulebook
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model(x)                         # warm the capture stream's allocations
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            got = model(x)
        for _ in range(4):
            got.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(got, want)
            assert torch.equal(model(x), want)   # eager in between
            torch.cuda.synchronize()
    assert scn.forward_pass_multiplyAdd_count > 0


def test_build_stream_and_single_stream_agree():
    """Rulebooks built on the library's own stream (beside the convolutions of the levels above)
    against the same forward passes with everything on the caller's stream: different scenes
    one after the other, Metadata objects dying while work is in flight, bit-identical results."""
    from sparseconvnet_amd import _lib
    L = _lib.lib()
    torch.manual_seed(10)
    m = 16
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 2, [m, 2 * m, 3 * m, 4 * m], True)).add(scn.BatchNormReLU(m)).add(scn.OutputLayer(3)).cuda().eval()
    randomise_bn(model, 10)
    scenes = []
    for i in range(6):
        coords = synthetic.room_scene(seed=9100 + i, target=30000 + 7000 * i, spatial=512, duplicate_fraction=0.2)
        scenes.append((torch.as_tensor(coords).cuda(), torch.rand((len(coords), 3), device="cuda")))
    inp = scn.InputLayer(3, 512, mode=4)

    def run_all():
        outs = []
        with torch.no_grad():
            for rep in range(2):
                for c, f in scenes:
                    outs.append(model(inp([c, f])))   # the previous scene's Metadata dies here
        torch.cuda.synchronize()
        return outs
    before = L.scn_set_build_stream(1)
    try:
        two = run_all()
        assert L.scn_set_build_stream(0) == 1
        one = run_all()
    finally:
        L.scn_set_build_stream(before)
    for a, b in zip(two, one):
        assert torch.equal(a, b)
    assert all(torch.isfinite(a).all() for a in two)


def test_input_batch_network_vs_oracle(oracle_built):
    """sparseconvnet/inputBatch.py's route into a network: points set one at a time and in
    blocks, an overwriting call, a sample cut from a dense tensor, rulebooks precomputed; the
    same calls on the CPU oracle, then the same module tree on both."""
    torch.manual_seed(5)
    rng = np.random.default_rng(5)
    model = hello_world_model().cuda().eval()
    randomise_bn(model, 6)
    size = model.input_spatial_size(torch.LongTensor([10, 10]))
    sp = size.numpy()
    p = cpu_path.CpuPath(2, "oracle")
    p.batch_begin(sp)

    def fill(batch):
        r = np.random.default_rng(7)
        batch.add_sample()
        pts = r.integers(0, sp[0], size=(300, 2))
        vec = r.normal(size=(300, 1)).astype(np.float32)
        for l, v in zip(pts[:20], vec[:20]):
            batch.set_location(torch.from_numpy(l), torch.from_numpy(v), False)
        batch.set_locations(torch.from_numpy(pts[20:]), torch.from_numpy(vec[20:]), False)
        batch.set_locations(torch.from_numpy(pts[:50]), torch.from_numpy(vec[100:150]), True)
        dense = torch.from_numpy(r.normal(size=(30, 40, 1)).astype(np.float32))
        batch.add_sample_from_tensor(dense, torch.LongTensor([int(sp[0]) - 20, 3]), 1.0)
        return pts, vec, dense.numpy()

    batch = scn.InputBatch(2, size)
    pts, vec, dense = fill(batch)
    p.batch_add_sample()
    p.batch_set_locations(pts, vec, False)
    p.batch_set_locations(pts[:50], vec[100:150], True)
    p.batch_add_sample_from_tensor(dense, [int(sp[0]) - 20, 3], 1.0)
    batch.precompute_metadata(3)
    p.generate_rulebooks(3)
    assert batch.batch_size() == 2 and batch.features.is_cuda
    assert (batch.get_spatial_locations().numpy() == p.spatial_locations(sp)).all()
    assert (batch.features.cpu().numpy() == p.batch_features()).all()
    with torch.no_grad():
        got = model(batch)
    want = oracle_model.run(model, p, oracle_model.CpuTensor(p.batch_features(), sp))
    checks.assert_close(got.cpu().numpy(), want, "network over an InputBatch")
    # without the precomputation the rulebooks are built on demand: same result
    again = scn.InputBatch(2, size)
    fill(again)
    with torch.no_grad():
        assert torch.equal(model(again), got)
    # points set after a look at the batch: the next look sees them
    extra = rng.integers(0, sp[0], size=(40, 2))
    extra_v = rng.normal(size=(40, 1)).astype(np.float32)
    batch.add_sample()
    batch.set_locations(torch.from_numpy(extra), torch.from_numpy(extra_v), False)
    p.batch_add_sample()
    p.batch_set_locations(extra, extra_v, False)
    assert batch.batch_size() == 3
    assert (batch.get_spatial_locations().numpy() == p.spatial_locations(sp)).all()
    assert (batch.features.cpu().numpy() == p.batch_features()).all()


def _network_rows_vs_oracle(model, dim, spatial, coords, planes, seed, out_planes, what):
    randomise_bn(model, seed)
    rng = np.random.default_rng(seed)
    feats = rng.uniform(-1, 1, size=(len(coords), planes)).astype(np.float32)
    inp_layer = scn.InputLayer(dim, spatial, mode=3)
    got, want, p = _run_both(model.eval(), inp_layer, [torch.as_tensor(coords), torch.as_tensor(feats)])
    out_sp = got.spatial_size.numpy()
    assert got.features.shape == (p.nactive(out_sp), out_planes), (got.features.shape, p.nactive(out_sp))
    rows = lambda loc: cpu_path.canon_rows(loc)  # noqa: E731
    checks.assert_close(got.features.cpu().numpy()[rows(got.get_spatial_locations().numpy())],
                        want.features[rows(p.spatial_locations(out_sp))], what)


def test_multiscale_vgg_vs_oracle(oracle_built):
    """SparseVggNet's multi-scale 'C' layers (networkArchitectures.py:33-130): branches one, two
    and three levels down by Convolution 3/2 and back up by Deconvolution 3/2, joined."""
    torch.manual_seed(11)
    model = scn.SparseVggNet(3, 3, [['C', 8, 4, 4, 4], 'MP', ['C', 8, 8], ['C3/2', 12]])
    spatial = model.input_spatial_size(torch.LongTensor([7, 7, 7]))
    assert (spatial == 31).all()
    coords = synthetic.scene_batch(seed=11000, batch=2, target=2500, spatial=31, n_boxes=5)
    _network_rows_vs_oracle(model, 3, 31, coords, 3, 11, 12, "multi-scale VGG")


def test_resnet_vs_oracle(oracle_built):
    """SparseResNet (networkArchitectures.py:132-200): identity, NetworkInNetwork and strided
    Convolution shortcuts."""
    torch.manual_seed(12)
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, 8, 3, False)).add(
        scn.SparseResNet(3, 8, [['basic', 8, 2, 1], ['basic', 12, 2, 1], ['basic', 16, 2, 2]]))
    spatial = model.input_spatial_size(torch.LongTensor([15, 15, 15]))
    assert (spatial == 31).all()
    coords = synthetic.scene_batch(seed=12000, batch=2, target=2500, spatial=31, n_boxes=5)
    _network_rows_vs_oracle(model, 3, 31, coords, 3, 12, 16, "ResNet")


@pytest.mark.parametrize("residual", [False, True])
def test_fully_convolutional_net_vs_oracle(oracle_built, residual):
    """FullyConvolutionalNet (networkArchitectures.py:259-312): every level's features unpooled
    to full resolution and joined."""
    torch.manual_seed(13)
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, 8, 3, False)).add(
        scn.FullyConvolutionalNet(3, 2, [8, 12, 16], residual_blocks=residual))
    coords = synthetic.scene_batch(seed=13000, batch=2, target=2500, spatial=32, n_boxes=5)
    _network_rows_vs_oracle(model, 3, 32, coords, 3, 13, 36, "fully convolutional net")


def test_dense_to_sparse_round_trip():
    """DenseToSparse (denseToSparse.py:13-67): rows are the non-zero cells in (sample, row-major)
    order; SparseToDense brings the dense tensor back; a convolution over the result agrees
    with the dense one at the active sites."""
    rng = np.random.default_rng(21)
    dense = rng.normal(size=(3, 4, 9, 7)).astype(np.float32)
    dense[rng.random((3, 1, 9, 7)).repeat(4, 1) < 0.6] = 0
    dense[2] = 0                                   # a sample without sites still counts
    x = scn.DenseToSparse(2)(torch.from_numpy(dense).cuda())
    cells = np.argwhere(np.abs(dense).sum(1) != 0)   # [n, 3]: sample, y, x
    assert x.batch_size() == 3 and (x.spatial_size == torch.LongTensor([9, 7])).all()
    assert (x.get_spatial_locations().numpy() == cells[:, [1, 2, 0]]).all()
    assert (x.features.cpu().numpy() == dense[cells[:, 0], :, cells[:, 1], cells[:, 2]]).all()
    assert (scn.SparseToDense(2, 4)(x).cpu().numpy() == dense).all()
    torch.manual_seed(21)
    conv = scn.SubmanifoldConvolution(2, 4, 5, 3, True).cuda()
    with torch.no_grad():
        y = conv(x)
    import bruteforce as bf
    loc = x.get_spatial_locations().numpy()
    want = bf.dense_subm_conv(loc, x.features.cpu().numpy(), conv.weight.detach().cpu().numpy(), (9, 7), 3, 3,
                              conv.bias.detach().cpu().numpy())
    checks.assert_close(y.features.cpu().numpy(), want, "convolution after DenseToSparse")


def test_pointwise_modules_and_dropout():
    torch.manual_seed(22)
    coords = torch.LongTensor([[1, 2, 0], [3, 3, 0], [0, 1, 1], [4, 4, 1]])
    feats = torch.randn(4, 6)
    x = scn.InputLayer(2, 6, mode=0)([coords, feats.cuda()])
    F = torch.nn.functional
    for module, fn in [(scn.ReLU(), F.relu), (scn.LeakyReLU(), lambda t: F.leaky_relu(t, 1 / 3)),
                       (scn.LeakyReLU(0.1), lambda t: F.leaky_relu(t, 0.1)), (scn.Tanh(), torch.tanh),
                       (scn.Sigmoid(), torch.sigmoid), (scn.ELU(), F.elu), (scn.SELU(), F.selu),
                       (scn.Dropout(0.25).eval(), lambda t: t * 0.75),
                       (scn.BatchwiseDropout(0.4).eval(), lambda t: t * 0.6)]:
        y = module(x)
        assert y.metadata is x.metadata and (y.spatial_size == x.spatial_size).all()
        assert torch.allclose(y.features.cpu(), fn(feats), rtol=1e-6, atol=1e-7), module
        assert (module.input_spatial_size(torch.LongTensor([5, 5])) == 5).all()
    kept = scn.Dropout(0.5).train()(x).features.cpu()
    assert ((kept == 0) | (kept == feats)).all()
    cols = scn.BatchwiseDropout(0.5).train()(x).features.cpu()
    assert all((cols[:, c] == 0).all() or (cols[:, c] == feats[:, c]).all() for c in range(6))
    bn_elu = scn.BatchNormELU(6).cuda().eval()
    randomise_bn(bn_elu, 22)
    with torch.no_grad():
        got = bn_elu(x).features.cpu()
    bn = bn_elu[0]
    want = F.elu((feats - bn.running_mean.cpu()) / torch.sqrt(bn.running_var.cpu() + bn.eps) * bn.weight.detach().cpu()
                 + bn.bias.detach().cpu())
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-5)


def test_tensor_utilities():
    """append_tensors, compare_sparse, AddCoords, concatenate / add_feature_planes
    (utils.py:53-108)."""
    rng = np.random.default_rng(23)

    def tensor(seed, batch, n):
        r = np.random.default_rng(seed)
        c = np.unique(np.concatenate([r.integers(0, 8, (n, 3)), r.integers(0, batch, (n, 1))], 1), axis=0)
        c = c[r.permutation(len(c))]
        f = r.normal(size=(len(c), 4)).astype(np.float32)
        return scn.InputLayer(3, 8, mode=0)([torch.from_numpy(c), torch.from_numpy(f).cuda()]), c, f

    a, ca, fa = tensor(1, 2, 150)
    b, cb, fb = tensor(2, 3, 100)
    ab = scn.append_tensors([a, b])
    assert ab.batch_size() == 5
    shifted = cb.copy()
    shifted[:, -1] += 2
    assert (ab.get_spatial_locations().numpy() == np.concatenate([ca, shifted])).all()
    assert (ab.features.cpu().numpy() == np.concatenate([fa, fb])).all()
    torch.manual_seed(23)
    conv = scn.SubmanifoldConvolution(3, 4, 6, 3, False).cuda()
    with torch.no_grad():   # samples do not see each other: the appended batch convolves like its parts
        assert torch.allclose(conv(ab).features, torch.cat([conv(a).features, conv(b).features]), rtol=1e-5,
                              atol=1e-6)
    # compare_sparse against a dictionary
    c, cc, fc = tensor(3, 2, 150)
    da = {tuple(k): v for k, v in zip(ca, fa.astype(np.float64))}
    dc = {tuple(k): v for k, v in zip(cc, fc.astype(np.float64))}
    assert set(da) & set(dc) and set(da) - set(dc) and set(dc) - set(da)
    err = sum((((da.get(k, 0) - dc.get(k, 0)) ** 2).sum() for k in set(da) | set(dc))) / len(set(da) | set(dc))
    assert abs(float(scn.compare_sparse(a, c)) - err) < 1e-4 * err
    assert float(scn.compare_sparse(a, a)) == 0
    # AddCoords: coordinates scaled to [-1, 1]
    with_coords = scn.AddCoords()(a)
    assert with_coords.features.shape == (len(ca), 7)
    assert np.allclose(with_coords.features.cpu().numpy()[:, 4:], ca[:, :3] / 3.5 - 1, atol=1e-6)
    assert (with_coords.features.cpu().numpy()[:, :4] == fa).all()
    # planes side by side / summed
    two = scn.concatenate_feature_planes([a, with_coords])
    assert two.features.shape == (len(ca), 11) and two.metadata is a.metadata
    assert torch.equal(scn.add_feature_planes([a, a, a]).features, a.features * 3)
    assert rng is not None


def test_reference_state_dict_reproduces_reference_output():
    """A state dict written by the reference's Python modules, loaded into the same network built
    from this package, gives the output the reference's CPU path computed for the fixture's input
    (tests/golden/make_state_dict_golden.py wrote both): checkpoints of the reference carry over."""
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    state = torch.load(os.path.join(here, "golden", "unet_state_dict.pth"), weights_only=True)
    io = np.load(os.path.join(here, "golden", "unet_state_dict_io.npz"))
    m = 8
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 1, [m, 2 * m, 3 * m], True)).add(scn.BatchNormReLU(m)).add(scn.OutputLayer(3))
    model.load_state_dict(state, strict=True)
    model = model.cuda().eval()
    with torch.no_grad():
        x = scn.InputLayer(3, 32, mode=4)([torch.as_tensor(io["coords"]), torch.as_tensor(io["feats"]).cuda()])
        got = model(x).cpu().numpy()
    checks.assert_close(got, io["out"], "output of the reference's checkpoint")
    for fuse in (False,):  # and with every batch norm as a pass of its own
        scn.fuse_batchnorm = fuse
        try:
            with torch.no_grad():
                x = scn.InputLayer(3, 32, mode=4)([torch.as_tensor(io["coords"]), torch.as_tensor(io["feats"]).cuda()])
                checks.assert_close(model(x).cpu().numpy(), io["out"], "unfused, output of the reference's checkpoint")
        finally:
            scn.fuse_batchnorm = True


def test_active_pooling_module():
    """ActivePooling at the end of a network: per-sample sums / means of the rows, and autograd
    through it (each row receives its sample's gradient, scaled by 1 / count when averaging)."""
    coords = synthetic.scene_batch(seed=5200, batch=3, target=2000, spatial=48, n_boxes=4, duplicate_fraction=0.0)
    feats = torch.randn((len(coords), 6), device="cuda", requires_grad=True)
    x = scn.InputLayer(3, 48, mode=3)([torch.as_tensor(coords), feats])
    sample = x.metadata.getSpatialLocations(x.spatial_size)[:, -1].cuda()
    for average in (False, True):
        y = scn.ActivePooling(3, average)(x)
        want = torch.zeros((3, 6), device="cuda").index_add_(0, sample, x.features.detach())
        count = torch.bincount(sample, minlength=3).float()
        if average:
            want = want / count[:, None]
        assert y.shape == (3, 6)
        checks.assert_close(y.detach().cpu().numpy(), want.cpu().numpy(), "active pooling module")
        g = torch.randn((3, 6), device="cuda")
        feats.grad = None
        (y * g).sum().backward()
        # mode 3 without repeated points: input rows are the level's rows
        expect = g[sample] / (count[sample][:, None] if average else 1.0)
        rows = x.metadata.getSpatialLocations(x.spatial_size)
        assert len(rows) == len(coords)
        checks.assert_close(feats.grad.cpu().numpy(), expect.cpu().numpy(), "active pooling module gradient")


def test_frozen_parameters_agree_and_follow_changes():
    """Eval-mode modules keep their packed weights and folded batch norms between calls: results
    are bit-identical with the cache on and off, a second call (which packs nothing) repeats the
    first, and a changed weight or statistic (in-place write, load_state_dict) is seen."""
    torch.manual_seed(12)
    m = 16
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 1, [m, 2 * m, 3 * m], True)).add(scn.BatchNormReLU(m)).add(scn.OutputLayer(3)).cuda().eval()
    randomise_bn(model, 12)
    coords = synthetic.room_scene(seed=9300, target=20000, spatial=256, duplicate_fraction=0.2)
    feats = torch.rand((len(coords), 3), device="cuda")
    layer = scn.InputLayer(3, 256, mode=4)

    def run():
        with torch.no_grad():
            return model(layer([torch.as_tensor(coords), feats])).clone()

    scn.frozen_parameters = False
    try:
        plain = run()
    finally:
        scn.frozen_parameters = True
    first, second = run(), run()
    assert torch.equal(first, plain) and torch.equal(second, plain)
    conv = [mod for mod in model.modules() if isinstance(mod, scn.SubmanifoldConvolution)][3]
    bn = [mod for mod in model.modules() if isinstance(mod, scn.BatchNormalization)][2]
    with torch.no_grad():
        conv.weight.mul_(1.5)
        bn.running_var.add_(0.25)
    changed = run()
    assert not torch.equal(changed, plain)
    scn.frozen_parameters = False
    try:
        assert torch.equal(run(), changed)
    finally:
        scn.frozen_parameters = True
    state = {k: v.clone() for k, v in model.state_dict().items()}
    with torch.no_grad():
        for p in model.parameters():
            p.mul_(0.5)
    assert not torch.equal(run(), changed)
    model.load_state_dict(state)
    assert torch.equal(run(), changed)
    with torch.no_grad():
        conv.weight.data.mul_(2.0)   # a write the version counter does not see ...
    scn.parameters_changed()         # ... announced by hand
    scn.frozen_parameters = False
    try:
        want = run()
    finally:
        scn.frozen_parameters = True
    assert torch.equal(run(), want) and not torch.equal(want, changed)


@pytest.mark.gpu
def test_frozen_parameters_follow_training_mode_batch_norm():
    """A training-mode forward updates the running statistics inside the library, through raw
    pointers.  The folded batch norms that eval-mode convolutions keep must notice: an eval pass,
    a train-mode forward without any optimiser step, and an eval pass again, which has to equal
    the result computed with nothing kept."""
    torch.manual_seed(13)
    m = 16
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 1, [m, 2 * m, 3 * m], False)).add(scn.BatchNormReLU(m)).add(scn.OutputLayer(3)).cuda().eval()
    randomise_bn(model, 13)
    for p in model.parameters():
        p.requires_grad_(False)  # a frozen backbone: no weight's version counter will move either
    coords = synthetic.room_scene(seed=9400, target=15000, spatial=256, duplicate_fraction=0.2)
    feats = torch.rand((len(coords), 3), device="cuda")
    layer = scn.InputLayer(3, 256, mode=4)

    def run():
        with torch.no_grad():
            return model(layer([torch.as_tensor(coords), feats])).clone()

    before = run()
    model.train()
    run()            # batch statistics; running_mean / running_var move
    model.eval()
    after = run()
    assert not torch.equal(after, before)
    scn.frozen_parameters = False
    try:
        want = run()
    finally:
        scn.frozen_parameters = True
    assert torch.equal(after, want)


@pytest.mark.parametrize("n_in,n_out", [(3, 16), (16, 16), (32, 64), (64, 32), (160, 160), (20, 24)])
def test_convolution_writes_into_columns_of_a_wider_matrix(n_in, n_out):
    """`out=` (scn_md_next_output_stride): the convolution fills a range of columns of a wider matrix
    and leaves the columns around it alone; the stride serves that one call."""
    coords = synthetic.scene_batch(seed=8100 + n_in, batch=2, target=9000, spatial=64, n_boxes=8)
    g = torch.Generator().manual_seed(n_in * 1000 + n_out)
    feats = torch.rand(len(coords), n_in, generator=g).cuda()
    t = scn.InputLayer(3, 64, mode=4)([torch.as_tensor(coords), feats])
    md, size, three, two = t.metadata, t.spatial_size, torch.LongTensor([3] * 3), torch.LongTensor([2] * 3)
    n = t.features.size(0)
    w = (torch.randn(27, 1, n_in, n_out, generator=g) * (2.0 / (27 * n_in)) ** 0.5).cuda()
    bias = torch.randn(n_out, generator=g).cuda()
    bn = (torch.randn(n_out, generator=g).cuda(), torch.rand(n_out, generator=g).cuda() + 0.5,
          torch.rand(n_out, generator=g).cuda() + 0.5, torch.randn(n_out, generator=g).cuda(), 1e-4, 0.1)
    for post in (None, bn):
        plain, _ = md.submanifoldConvolution(size, three, t.features, w, bias, post=post, want_macs=False)
        wide = torch.full((n, n_out + 24), 7.0, device="cuda")
        got, _ = md.submanifoldConvolution(size, three, t.features, w, bias, post=post, want_macs=False,
                                           out=wide[:, 8:8 + n_out])
        assert got.data_ptr() == wide[:, 8:].data_ptr()
        checks.assert_close(wide[:, 8:8 + n_out].cpu().numpy(), plain.cpu().numpy(), "columns of the wide matrix")
        assert (wide[:, :8] == 7.0).all() and (wide[:, 8 + n_out:] == 7.0).all()
        again, _ = md.submanifoldConvolution(size, three, t.features, w, bias, post=post, want_macs=False)
        assert again.is_contiguous() and torch.equal(again, plain), "the stride must not outlive its call"
        # `second=`: the plain output as before, and beside it the raw output under another batch norm
        raw, _ = md.submanifoldConvolution(size, three, t.features, w, bias, want_macs=False)
        mean2, var2, g2, b2 = bn[1] - 0.7, bn[1] + 0.1, bn[3] * 0.5 + 1.0, bn[0]
        want2 = (raw - mean2) / torch.sqrt(var2 + 1e-4) * g2 + b2
        want2 = torch.where(want2 > 0, want2, 0.2 * want2)
        wide2 = torch.full((n, n_out + 12), 5.0, device="cuda")
        got, _ = md.submanifoldConvolution(size, three, t.features, w, bias, post=post, want_macs=False,
                                           second=((mean2, var2, g2, b2, 1e-4, 0.2), wide2[:, 4:4 + n_out]))
        checks.assert_close(got.cpu().numpy(), plain.cpu().numpy(), "plain output beside a second one")
        checks.assert_close(wide2[:, 4:4 + n_out].cpu().numpy(), want2.cpu().numpy(), "second output")
        assert (wide2[:, :4] == 5.0).all() and (wide2[:, 4 + n_out:] == 5.0).all()
        again, _ = md.submanifoldConvolution(size, three, t.features, w, bias, post=post, want_macs=False)
        assert torch.equal(again, plain), "the second output must not outlive its call"
    # strided and transposed convolutions (8 taps): down to the coarse level and back up
    half = (size - 2) // 2 + 1
    w2 = (torch.randn(8, 1, n_in, n_out, generator=g) * (2.0 / (8 * n_in)) ** 0.5).cuda()
    down, _ = md.convolution(size, half, two, two, t.features, w2, None, want_macs=False)
    wide = torch.full((down.size(0), n_out + 16), -3.0, device="cuda")
    md.convolution(size, half, two, two, t.features, w2, None, want_macs=False, out=wide[:, 16:])
    checks.assert_close(wide[:, 16:].cpu().numpy(), down.cpu().numpy(), "strided convolution into columns")
    assert (wide[:, :16] == -3.0).all()
    w3 = (torch.randn(8, 1, n_out, n_in, generator=g) * (2.0 / (8 * n_out)) ** 0.5).cuda()
    up, _ = md.deconvolution(half, size, two, two, down, w3, None, want_macs=False)
    wide = torch.full((n, n_in + 8), 2.0, device="cuda")
    md.deconvolution(half, size, two, two, down, w3, None, want_macs=False, out=wide[:, :n_in])
    checks.assert_close(wide[:, :n_in].cpu().numpy(), up.cpu().numpy(), "transposed convolution into columns")
    assert (wide[:, n_in:] == 2.0).all()


def test_unet_level_joins_without_a_pass_over_the_joined_matrix():
    """ConcatTable + JoinTable + eval-mode batch norm (every level of a U-Net): the Deconvolution
    that ends the inner branch normalises its own planes into its columns of the joined matrix.
    Same result as the three modules one after the other, and the path is the one taken."""
    from sparseconvnet_amd import layers
    torch.manual_seed(11)
    m = 16
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 2, [m, 2 * m, 3 * m], False, leakiness=0.1)).add(scn.BatchNormReLU(m)).add(
        scn.OutputLayer(3)).cuda().eval()
    randomise_bn(model, 11)
    coords = synthetic.scene_batch(seed=11000, batch=2, target=8000, spatial=64, n_boxes=8, duplicate_fraction=0.2)
    feats = torch.rand(len(coords), 3).cuda()
    inp_layer = scn.InputLayer(3, 64, mode=4)
    orig, taken = layers.concat_join_batchnorm, []
    orig_plan, planned = layers.skip_join_plan, []

    def counting(table, bn, input, prefilled=None):
        r = orig(table, bn, input, prefilled)
        taken.append((r is not None, prefilled is not None))
        return r

    def counting_plan(conv, mods, input):
        r = orig_plan(conv, mods, input)
        planned.append(r is not None)
        return r
    outs = []
    try:
        # both halves by their producers; the transposed convolution's half only; a pass over the joined matrix
        for fn, plan in ((counting, counting_plan), (counting, lambda conv, mods, input: None),
                         (lambda table, bn, input, prefilled=None: None, lambda conv, mods, input: None)):
            layers.concat_join_batchnorm, layers.skip_join_plan = fn, plan
            with torch.no_grad():
                outs.append(model(inp_layer([torch.as_tensor(coords), feats])).cpu().numpy())
    finally:
        layers.concat_join_batchnorm, layers.skip_join_plan = orig, orig_plan
    # two levels with an inner branch, twice; the first time the skip halves were there already
    assert taken == [(True, True)] * 2 + [(True, False)] * 2, taken
    assert planned.count(True) == 2, planned
    checks.assert_close(outs[0], outs[2], "joined by the producers vs joined by a pass")
    checks.assert_close(outs[1], outs[2], "transposed convolution's half by its producer vs joined by a pass")
    # with gradients enabled the modules run one after the other
    taken.clear()
    layers.concat_join_batchnorm = counting
    try:
        model(inp_layer([torch.as_tensor(coords), feats]))
    finally:
        layers.concat_join_batchnorm = orig
    assert taken == [(False, False)] * 2, taken


def test_frozen_parameters_of_a_wide_layer_do_not_grow():
    """More than 256 output planes run as column ranges over a scratch copy of the weights.  The
    frozen set keys those ranges by where they lie in the module's weights, not by the scratch
    address: over a stream of scenes (a new Metadata each, scratch at changing addresses) the
    results stay those of the uncached path and the memory the library holds stops growing."""
    import ctypes as C
    from sparseconvnet_amd import _lib
    torch.manual_seed(14)
    conv = scn.SubmanifoldConvolution(3, 16, 320, 3, True).cuda().eval()
    with torch.no_grad():
        conv.bias.normal_()
    layer = scn.InputLayer(3, 64, mode=4)
    L = _lib.lib()

    def live():
        torch.cuda.synchronize()
        a, b = C.c_int64(0), C.c_int64(0)
        _lib.check(L.scn_cache_stats(C.byref(a), C.byref(b), None, None))
        return a.value

    def run(seed):
        coords = synthetic.scene_batch(seed=seed, batch=1, target=3000 + 500 * (seed % 3), spatial=64, n_boxes=6)
        feats = torch.rand((len(coords), 16), device="cuda", generator=torch.Generator(device="cuda").manual_seed(seed))
        with torch.no_grad():
            return conv(layer([torch.as_tensor(coords), feats])).features.clone()

    scn.frozen_parameters = False
    try:
        want = [run(s) for s in range(3)]
    finally:
        scn.frozen_parameters = True
    sizes = []
    for rep in range(4):
        for s in range(3):
            assert torch.equal(run(s), want[s]), (rep, s)
        sizes.append(live())
    assert sizes[1] == sizes[2] == sizes[3], sizes
