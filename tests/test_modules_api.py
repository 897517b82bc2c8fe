"""The Python module API against what the reference's modules promise (constructor
signatures, attribute names, parameter shapes and initialisation, spatial-size arithmetic,
repr strings, state_dict layout).  No GPU needed.  Citations: reference sparseconvnet/*.py."""
import math

import pytest
import torch

import sparseconvnet_amd as scn


def hello_world_model():
    # examples/hello-world.py:19-30
    return scn.Sequential().add(
        scn.SparseVggNet(2, 1, [['C', 8], ['C', 8], ['MP', 3, 2], ['C', 16], ['C', 16], ['MP', 3, 2],
                                ['C', 24], ['C', 24], ['MP', 3, 2]])
    ).add(scn.SubmanifoldConvolution(2, 24, 32, 3, False)).add(scn.BatchNormReLU(32)).add(scn.SparseToDense(2, 32))


def test_exports():
    for name in ["SubmanifoldConvolution", "ValidConvolution", "Convolution", "Deconvolution",
                 "BatchNormalization", "BatchNormReLU", "BatchNormLeakyReLU", "MaxPooling", "InputLayer",
                 "OutputLayer", "SparseToDense", "Metadata", "SparseConvNetTensor", "Sequential", "ConcatTable",
                 "JoinTable", "AddTable", "Identity", "SparseVggNet", "UNet", "toLongTensor", "optionalTensor",
                 "NetworkInNetwork", "AveragePooling", "UnPooling", "BLInputLayer", "BLOutputLayer", "InputBatch", "SparseResNet",
                 "FullyConvolutionalNet", "DenseToSparse", "InputLayerInput", "ReLU", "LeakyReLU", "Tanh",
                 "Sigmoid", "ELU", "SELU", "BatchNormELU", "Dropout", "BatchwiseDropout", "AddCoords",
                 "append_tensors", "compare_sparse", "concatenate_feature_planes", "add_feature_planes",
                 "CheckpointedSequential"]:
        assert hasattr(scn, name), name
    assert scn.forward_pass_multiplyAdd_count == 0 and scn.forward_pass_hidden_states == 0


def test_conv_parameters_and_repr():
    # submanifoldConvolution.py:15-28,45-56; convolution.py:14-29,53-67
    c = scn.SubmanifoldConvolution(3, 16, 32, 3, False)
    assert tuple(c.weight.shape) == (27, 1, 16, 32) and not hasattr(c, 'bias')
    assert c.filter_volume == 27 and c.filter_size.tolist() == [3, 3, 3] and c.dimension == 3
    assert repr(c) == 'SubmanifoldConvolution 16->32 C3'
    assert repr(scn.SubmanifoldConvolution(3, 4, 4, [3, 1, 3], True)) == 'SubmanifoldConvolution 4->4 C(3,1,3)'
    g = scn.SubmanifoldConvolution(2, 8, 12, 3, True, groups=2)
    assert tuple(g.weight.shape) == (9, 2, 4, 6) and tuple(g.bias.shape) == (12,) and (g.bias == 0).all()
    d = scn.Convolution(3, 32, 64, 2, 2, False)
    assert tuple(d.weight.shape) == (8, 1, 32, 64) and repr(d) == 'Convolution 32->64 C2/2'
    assert repr(scn.Convolution(2, 1, 1, [3, 2], [2, 1], False)) == 'Convolution 1->1 C(3,2)/(2,1)'
    u = scn.Deconvolution(3, 64, 32, 2, 2, False)
    assert tuple(u.weight.shape) == (8, 1, 64, 32) and repr(u) == 'Deconvolution 64->32 C2/2'
    assert issubclass(scn.ValidConvolution, scn.SubmanifoldConvolution)


def test_weight_initialisation_scale():
    # std = sqrt(2 * groups / (nIn * filter_volume)), submanifoldConvolution.py:23-26
    torch.manual_seed(0)
    c = scn.SubmanifoldConvolution(3, 64, 64, 3, False)
    want = math.sqrt(2.0 / (64 * 27))
    assert abs(c.weight.std().item() / want - 1) < 0.02 and abs(c.weight.mean().item()) < 0.1 * want


def test_spatial_size_arithmetic():
    t = torch.LongTensor
    assert scn.Convolution(3, 1, 1, 2, 2, False).input_spatial_size(t([64] * 3)).tolist() == [128] * 3
    assert scn.Convolution(2, 1, 1, 3, 2, False).input_spatial_size(t([7, 7])).tolist() == [15, 15]
    assert scn.MaxPooling(2, 3, 2).input_spatial_size(t([8, 8])).tolist() == [17, 17]
    assert scn.SubmanifoldConvolution(2, 1, 1, 3, False).input_spatial_size(t([9, 9])).tolist() == [9, 9]
    # hello world: three MP3/2 need 8k+7 (README "Output is 2x32x10x10" for input 87)
    m = hello_world_model()
    assert m.input_spatial_size(t([10, 10])).tolist() == [87, 87]
    assert m.input_spatial_size(t([8, 8])).tolist() == [71, 71]


def test_pooling_modules():
    # averagePooling.py:21-66, unPooling.py:59-96
    a = scn.AveragePooling(3, 3, 2)
    assert repr(a) == 'AveragePooling3/2' and (a.input_spatial_size(torch.LongTensor([7, 7, 7])) == 15).all()
    assert repr(scn.AveragePooling(2, [3, 2], [2, 1])) == 'AveragePooling(3,2)/(2,1)'
    u = scn.UnPooling(3, 2, 2)
    assert repr(u) == 'UnPooling2/2' and (u.input_spatial_size(torch.LongTensor([4, 4, 4])) == 8).all()
    assert u.nFeaturesToDrop == 0 and len(list(u.parameters())) == 0


def test_bn_modules():
    # batchNormalization.py:13-91
    b = scn.BatchNormalization(5)
    assert b.eps == 1e-4 and b.momentum == 0.99 and b.leakiness == 1 and b.affine
    assert (b.running_mean == 0).all() and (b.running_var == 1).all() and (b.weight == 1).all()
    assert sorted(b.state_dict()) == ['bias', 'running_mean', 'running_var', 'weight']
    assert scn.BatchNormReLU(4).leakiness == 0
    assert scn.BatchNormLeakyReLU(4).leakiness == 0.333
    assert repr(scn.BatchNormReLU(32)) == 'BatchNormReLU(32,eps=0.0001,momentum=0.99,affine=True)'
    assert repr(scn.BatchNormLeakyReLU(8, leakiness=0)) == \
        'BatchNormLeakyReLU(8,eps=0.0001,momentum=0.99,affine=True,leakiness=0)'
    assert repr(scn.BatchNormalization(3)) == 'BatchNorm(3,eps=0.0001,momentum=0.99,affine=True,leakiness=1)'


def test_containers():
    s = scn.Sequential().add(scn.Identity()).add(scn.BatchNormReLU(3))
    assert len(s) == 2 and isinstance(s[1], scn.BatchNormReLU)
    s2 = s + scn.Sequential().add(scn.Identity())
    assert len(s2) == 3
    s.insert(0, scn.MaxPooling(2, 3, 2))
    assert isinstance(s[0], scn.MaxPooling) and len(s) == 3
    ct = scn.ConcatTable().add(scn.Identity()).add(scn.Identity())
    assert len(ct) == 2
    a = scn.SparseConvNetTensor(torch.ones(3, 2), None, torch.LongTensor([4, 4]))
    b = scn.SparseConvNetTensor(2 * torch.ones(3, 5), None, torch.LongTensor([4, 4]))
    j = scn.JoinTable()(ct(a)[:1] + [b])
    assert tuple(j.features.shape) == (3, 7) and j.spatial_size is a.spatial_size
    assert (scn.AddTable()([a, a]).features == 2).all()


def test_unet_structure_and_state_dict():
    # networkArchitectures.py:203-257 with examples/ScanNet/unet.py:25-38 (m=32, reps=2, 7 levels)
    m = 32
    planes = [m * i for i in range(1, 8)]
    u = scn.UNet(3, 2, planes, False)
    convs = [x for x in u.modules() if isinstance(x, scn.SubmanifoldConvolution)]
    downs = [x for x in u.modules() if isinstance(x, scn.Convolution)]
    ups = [x for x in u.modules() if isinstance(x, scn.Deconvolution)]
    bns = [x for x in u.modules() if isinstance(x, scn.BatchNormalization)]
    assert len(convs) == 2 * 7 + 2 * 6 and len(downs) == 6 and len(ups) == 6 and len(bns) == 26 + 12
    assert [(c.nIn, c.nOut) for c in downs] == [(planes[i], planes[i + 1]) for i in range(6)]
    assert sorted((c.nIn, c.nOut) for c in ups) == sorted((planes[i + 1], planes[i]) for i in range(6))
    assert (64, 32) in [(c.nIn, c.nOut) for c in convs] and (448, 224) not in [(c.nIn, c.nOut) for c in convs]
    assert all(b.leakiness == 0 for b in bns)
    # first block, as torch names it: sequential indices nest exactly as in the reference
    sd = u.state_dict()
    assert tuple(sd['0.1.weight'].shape) == (27, 1, 32, 32) and '0.0.running_mean' in sd
    assert tuple(sd['2.1.1.weight'].shape) == (8, 1, 32, 64)      # Convolution 32->64 C2/2
    assert tuple(sd['2.1.4.weight'].shape) == (8, 1, 64, 32)      # Deconvolution 64->32 C2/2
    assert tuple(sd['4.1.weight'].shape) == (27, 1, 64, 32)       # first block after the join


def test_residual_unet_structure():
    # networkArchitectures.py:222-230: a NetworkInNetwork only where a block changes the plane count
    u = scn.UNet(3, 2, [8, 16, 24], residual_blocks=True, n_input_planes=5)
    nins = [x for x in u.modules() if isinstance(x, scn.NetworkInNetwork)]
    assert sorted((n.nIn, n.nOut) for n in nins) == [(5, 8), (16, 8), (32, 16)]
    assert all(not hasattr(n, 'bias') and tuple(n.weight.shape) == (n.nIn, n.nOut) for n in nins)
    adds = [x for x in u.modules() if isinstance(x, scn.AddTable)]
    convs = [x for x in u.modules() if isinstance(x, scn.SubmanifoldConvolution)]
    assert len(adds) == 2 * 3 + 2 * 2 and len(convs) == 2 * len(adds)
    sd = u.state_dict()
    # block 0: ConcatTable(NetworkInNetwork, Sequential(BN, conv, BN, conv)), then AddTable
    assert tuple(sd['0.0.weight'].shape) == (5, 8)
    assert tuple(sd['0.1.1.weight'].shape) == (27, 1, 5, 8) and tuple(sd['0.1.3.weight'].shape) == (27, 1, 8, 8)
    # block 1 keeps the plane count: Identity has no parameters
    assert '2.0.weight' not in sd and tuple(sd['2.1.1.weight'].shape) == (27, 1, 8, 8)
    n = scn.NetworkInNetwork(6, 4, True)
    assert tuple(n.bias.shape) == (4,) and (n.bias == 0).all()
    assert abs(scn.NetworkInNetwork(400, 300, False).weight.std().item() - (2.0 / 400) ** 0.5) < 2e-3


def test_checkpoint_round_trip(tmp_path):
    # utils.py:138-177: file naming, newest-epoch lookup, pruning of non-power-of-two epochs
    torch.manual_seed(3)
    a = scn.UNet(3, 1, [4, 8], False)
    stem = str(tmp_path / "exp")
    assert scn.checkpoint_restore(a, stem, "unet", use_cuda=False) == 1
    for epoch in (1, 2, 3, 4, 5):
        scn.checkpoint_save(a, stem, "unet", epoch, use_cuda=False)
    kept = sorted(f.name for f in tmp_path.iterdir())
    assert kept == ["exp-%09d-unet.pth" % e for e in (1, 2, 4, 5)]
    b = scn.UNet(3, 1, [4, 8], False)
    assert scn.checkpoint_restore(b, stem, "unet", use_cuda=False) == 6
    for (ka, va), (kb, vb) in zip(a.state_dict().items(), b.state_dict().items()):
        assert ka == kb and torch.equal(va, vb)
    assert scn.is_power2(8) and not scn.is_power2(6) and not scn.is_power2(0)


def test_input_batch_collects_on_the_host():
    # sparseconvnet/inputBatch.py:22-70: the calls and their old names; nothing touches the GPU
    # until the features or the metadata are looked at
    b = scn.InputBatch(2, [8, 6])
    with pytest.raises(RuntimeError):
        b.set_locations(torch.LongTensor([[1, 2]]), torch.FloatTensor([[1.0]]))
    b.add_sample()
    b.set_location(torch.LongTensor([1, 2]), torch.FloatTensor([1.0]))
    with pytest.raises(AssertionError):
        b.set_location(torch.LongTensor([1, 6]), torch.FloatTensor([1.0]))
    with pytest.raises(AssertionError):
        b.set_locations(torch.LongTensor([[8, 0, 0]]), torch.FloatTensor([[1.0]]))
    b.set_locations(torch.LongTensor([[0, 0, 3], [7, 5, 1]]), torch.FloatTensor([[2.0], [3.0]]), True)
    b.addSample()
    b.setLocations(torch.LongTensor([[4, 4]]), torch.FloatTensor([[4.0]]))
    t = torch.zeros(3, 3, 1)
    t[0, 0, 0], t[2, 2, 0], t[1, 1, 0] = 5.0, -6.0, 0.5
    b.add_sample_from_tensor(t, torch.LongTensor([5, 3]), threshold=1)
    assert b._samples == 6
    assert torch.cat(b._coords).tolist() == [[1, 2, 0], [0, 0, 3], [7, 5, 1], [4, 4, 4], [5, 3, 5], [7, 5, 5]]
    assert torch.cat(b._vectors).flatten().tolist() == [1.0, 2.0, 3.0, 4.0, 5.0, -6.0]
    assert b._overwrite == [(1, False), (2, True), (1, False), (2, False)]
    for name in ("addSample", "setLocation", "setLocation_", "setLocations", "setLocations_",
                 "addSampleFromTensor", "precomputeMetadata", "precompute_metadata"):
        assert callable(getattr(b, name))
    if not torch.cuda.is_available():
        with pytest.raises(Exception):
            b.features


def test_remaining_builders_structure():
    # networkArchitectures.py:33-130: ['C', a, b, c] = 3^d convolution beside branches one and two
    # levels down; planes add up; module order inside the branches
    m = scn.SparseVggNet(2, 3, [['C', 8, 4, 6]])
    table, join, bn = m[0], m[1], m[2]
    assert isinstance(table, scn.ConcatTable) and isinstance(join, scn.JoinTable) and bn.nPlanes == 18
    kinds = [type(x).__name__ for x in table[2]]
    assert kinds == ["Convolution", "BatchNormReLU", "SubmanifoldConvolution", "BatchNormReLU"] * 2 + [
        "Deconvolution", "BatchNormReLU", "SubmanifoldConvolution", "BatchNormReLU", "Deconvolution"]
    assert [type(x).__name__ for x in table[1]] == ["Convolution", "BatchNormReLU", "SubmanifoldConvolution",
                                                    "BatchNormReLU", "Deconvolution"]
    assert (m.input_spatial_size(torch.LongTensor([7, 7])) == 7).all()
    # networkArchitectures.py:132-200: state-dict names of a two-stage ResNet
    r = scn.SparseResNet(3, 4, [['basic', 8, 2, 1], ['basic', 16, 1, 2]])
    keys = [k for k in r.state_dict() if k.endswith("weight") and "running" not in k]
    assert keys == ['0.weight', '1.0.0.weight', '1.0.1.weight', '1.0.2.weight', '1.1.weight',
                    '3.0.0.weight', '3.0.1.weight', '3.0.2.weight', '3.0.3.weight',
                    '5.weight', '6.0.0.weight', '6.0.1.weight', '6.0.2.weight', '6.1.weight', '8.weight']
    assert isinstance(r[1][1], scn.NetworkInNetwork) and isinstance(r[3][1], scn.Identity)
    assert isinstance(r[6][1], scn.Convolution) and isinstance(r[6][0][0], scn.Convolution)
    assert (r.input_spatial_size(torch.LongTensor([5, 5, 5])) == 11).all()
    # networkArchitectures.py:259-312
    f = scn.FullyConvolutionalNet(3, 1, [8, 16, 24])
    assert isinstance(f[1][1][3], scn.UnPooling) and isinstance(f[2], scn.JoinTable)
    assert (f.input_spatial_size(torch.LongTensor([8, 8, 8])) == 8).all()


def test_no_cpu_fallback():
    from sparseconvnet_amd._lib import ScnError
    layer = scn.InputLayer(2, 8, mode=3)
    coords = torch.LongTensor([[1, 2, 0], [3, 4, 0]])
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises((ScnError, RuntimeError, AssertionError)):
        layer([coords, torch.ones(2, 1)])
    with pytest.raises(ScnError):
        scn.metadata.batchNormEval(torch.ones(2, 3), torch.zeros(3), torch.ones(3), None, None, 1e-4, 0)


def test_reference_state_dict_loads_strictly():
    """tests/golden/unet_state_dict.pth was written by the reference's own Python modules
    (tests/golden/make_state_dict_golden.py): the same constructor calls on this package give a
    model whose state dict has exactly those keys, in that order, with those shapes, and
    load_state_dict(strict=True) accepts the file (what sparseconvnet/utils.py:138-177 does with a
    checkpoint)."""
    import os
    import torch
    sys_path_root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    state = torch.load(os.path.join(sys_path_root, "tests", "golden", "unet_state_dict.pth"), weights_only=True)
    m = 8
    model = scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 1, [m, 2 * m, 3 * m], True)).add(scn.BatchNormReLU(m)).add(scn.OutputLayer(3))
    own = model.state_dict()
    assert list(own) == list(state)
    assert [tuple(v.shape) for v in own.values()] == [tuple(v.shape) for v in state.values()]
    assert all(v.dtype == state[k].dtype for k, v in own.items())
    result = model.load_state_dict(state, strict=True)
    assert not result.missing_keys and not result.unexpected_keys
