"""Runs a sparseconvnet_amd module tree on the CPU oracle: walks the containers and applies
the oracle's op for every layer with that layer's own parameters.  Used to check whole
networks (the VGG and U-Net configurations) end to end against the library."""
import numpy as np

import sparseconvnet_amd as scn


class CpuTensor:
    def __init__(self, features, spatial):
        self.features = features
        self.spatial = np.asarray(spatial, np.int64)


def _np(t):
    return t.detach().cpu().numpy()


def run(module, path, x):
    """path: oracle.cpu_path.CpuPath holding the metadata; x: CpuTensor or, for an InputLayer,
    the [coords, features] pair."""
    if isinstance(module, scn.InputLayer):
        coords, feats = _np(x[0]), _np(x[1]).astype(np.float32)
        sp = _np(module.spatial_size)
        path.input_layer(sp, coords, 0 if len(x) == 2 else x[2], module.mode)
        return CpuTensor(path.input_fwd(feats), sp)
    if isinstance(module, scn.BLInputLayer):
        coords, feats = _np(x[0]), _np(x[1]).astype(np.float32)
        sp = _np(module.spatial_size)
        path.bl_input_layer(sp, coords, module.mode)
        return CpuTensor(path.bl_input_fwd(feats), sp)
    if isinstance(module, scn.BLOutputLayer):
        return path.bl_output_fwd(x.features)
    if isinstance(module, scn.OutputLayer):
        return path.output_fwd(x.features)
    if isinstance(module, scn.SubmanifoldConvolution):
        b = _np(module.bias) if hasattr(module, 'bias') else None
        y, _ = path.subm_conv(x.spatial, _np(module.filter_size), x.features, _np(module.weight), b)
        return CpuTensor(y, x.spatial)
    if isinstance(module, scn.Convolution):
        fs, st = _np(module.filter_size), _np(module.filter_stride)
        out_sp = (x.spatial - fs) // st + 1
        b = _np(module.bias) if hasattr(module, 'bias') else None
        y, _ = path.conv(x.spatial, out_sp, fs, st, x.features, _np(module.weight), b)
        return CpuTensor(y, out_sp)
    if isinstance(module, scn.Deconvolution):
        fs, st = _np(module.filter_size), _np(module.filter_stride)
        out_sp = (x.spatial - 1) * st + fs
        b = _np(module.bias) if hasattr(module, 'bias') else None
        y, _ = path.deconv(x.spatial, out_sp, fs, st, x.features, _np(module.weight), b)
        return CpuTensor(y, out_sp)
    if isinstance(module, scn.NetworkInNetwork):
        b = _np(module.bias) if hasattr(module, 'bias') else None
        y, _ = path.nin(x.features, _np(module.weight), b)
        return CpuTensor(y, x.spatial)
    if isinstance(module, scn.AveragePooling):
        ps, st = _np(module.pool_size), _np(module.pool_stride)
        out_sp = (x.spatial - ps) // st + 1
        return CpuTensor(path.avgpool(x.spatial, out_sp, ps, st, x.features, module.nFeaturesToDrop), out_sp)
    if isinstance(module, scn.UnPooling):
        ps, st = _np(module.pool_size), _np(module.pool_stride)
        out_sp = (x.spatial - 1) * st + ps
        return CpuTensor(path.unpool(x.spatial, out_sp, ps, st, x.features, module.nFeaturesToDrop), out_sp)
    if isinstance(module, scn.MaxPooling):
        ps, st = _np(module.pool_size), _np(module.pool_stride)
        out_sp = (x.spatial - ps) // st + 1
        return CpuTensor(path.maxpool(x.spatial, out_sp, ps, st, x.features, module.nFeaturesToDrop), out_sp)
    if isinstance(module, scn.BatchNormalization):
        if x.features.size == 0:
            return x
        w = _np(module.weight) if hasattr(module, 'weight') else None
        b = _np(module.bias) if hasattr(module, 'bias') else None
        y = path.bn_eval(x.features, _np(module.running_mean), _np(module.running_var), w, b, module.eps,
                         module.leakiness)
        return CpuTensor(y, x.spatial)
    if isinstance(module, scn.SparseToDense):
        return path.s2d(x.spatial, x.features)
    if isinstance(module, scn.Identity):
        return x
    if isinstance(module, scn.ConcatTable):
        return [run(m, path, x) for m in module._modules.values()]
    if isinstance(module, scn.JoinTable):
        return CpuTensor(np.concatenate([t.features for t in x], 1), x[0].spatial)
    if isinstance(module, scn.AddTable):
        return CpuTensor(sum(t.features for t in x), x[0].spatial)
    if isinstance(module, scn.Sequential):
        for m in module._modules.values():
            x = run(m, path, x)
        return x
    raise TypeError("no oracle op for %r" % type(module))
