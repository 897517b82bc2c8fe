"""Small helpers shared by the modules (same names and meaning as the reference's
sparseconvnet/utils.py:11-26)."""
import glob
import os

import torch


def toLongTensor(dimension, x):
    """A CPU LongTensor of `dimension` sizes from an int, a list/tuple or a LongTensor."""
    if isinstance(x, torch.Tensor):
        if x.dtype != torch.int64 or x.is_cuda:
            x = x.detach().cpu().long()
        assert x.numel() == dimension
        return x
    if isinstance(x, (list, tuple)):
        assert len(x) == dimension
        return torch.tensor([int(v) for v in x], dtype=torch.int64)
    return torch.full((dimension,), int(x), dtype=torch.int64)


_EMPTY = torch.Tensor()
_REGISTRIES = ('_parameters', '_buffers', '_modules')


def optionalTensor(module, name):
    """module.<name> if it exists, else an empty tensor (how the reference passes 'no bias').
    Called for every bias and batch-norm weight of every module call: a Module's registries are
    looked at directly (hasattr on a Module without the attribute goes through an exception), and
    the empty tensor is one shared object, which nobody writes to."""
    d = getattr(module, '__dict__', None)
    if d is not None:
        if name in d:
            return d[name]
        for reg in _REGISTRIES:
            r = d.get(reg)
            if r is not None and name in r:
                return r[name]
        if not hasattr(type(module), name):
            return _EMPTY
    return getattr(module, name) if hasattr(module, name) else _EMPTY


def optionalTensorReturn(a):
    return a if a.numel() else None


def prepare_BLInput(batch):
    """utils.py:127-136: pads a list of (locations [n_i, d], features [n_i, planes]) samples
    to one [batch, max n_i, d] location tensor (filled up with -1 = empty) and one
    [batch, max n_i, planes] feature tensor (filled up with zeros) for BLInputLayer."""
    with torch.no_grad():
        longest = max(loc.size(0) for loc, _ in batch)
        loc0, feat0 = batch[0]
        locations = torch.full((len(batch), longest, loc0.size(1)), -1, dtype=torch.int64)
        features = torch.zeros(len(batch), longest, feat0.size(1))
        for i, (loc, feat) in enumerate(batch):
            locations[i, :loc.size(0)] = loc
            features[i, :feat.size(0)] = feat
    return [locations, features]


def is_power2(num):
    """utils.py:157-158."""
    return num != 0 and ((num & (num - 1)) == 0)


def checkpoint_restore(model, exp_name, name2, use_cuda=True, epoch=0):
    """utils.py:138-155: loads `<exp_name>-<epoch, 9 digits>-<name2>.pth` (the newest one when
    epoch is 0) into the model and returns the epoch to continue with; 1 when there is none.
    The state dict is read with weights_only=True: parameter and buffer tensors only."""
    if use_cuda:
        model.cpu()
    if epoch > 0:
        f = exp_name + '-%09d-' % epoch + name2 + '.pth'
        assert os.path.isfile(f)
        print('Restore from ' + f)
        model.load_state_dict(torch.load(f, weights_only=True))
    else:
        found = sorted(glob.glob(exp_name + '-*-' + name2 + '.pth'))
        if len(found) > 0:
            f = found[-1]
            print('Restore from ' + f)
            model.load_state_dict(torch.load(f, weights_only=True))
            epoch = int(f[len(exp_name) + 1:-len(name2) - 5])
    if use_cuda:
        model.cuda()
    return epoch + 1


def checkpoint_save(model, exp_name, name2, epoch, use_cuda=True):
    """utils.py:166-177: saves the state dict and removes the previous epoch's file unless its
    number is a power of two."""
    f = exp_name + '-%09d-' % epoch + name2 + '.pth'
    model.cpu()
    torch.save(model.state_dict(), f)
    if use_cuda:
        model.cuda()
    epoch = epoch - 1
    f = exp_name + '-%09d-' % epoch + name2 + '.pth'
    if os.path.isfile(f) and not is_power2(epoch):
        os.remove(f)


def concatenate_feature_planes(input):
    """utils.py:53-58: tensors over the same sites, planes side by side."""
    from .tensor import SparseConvNetTensor
    return SparseConvNetTensor(torch.cat([i.features for i in input], 1), input[0].metadata, input[0].spatial_size)


def add_feature_planes(input):
    """utils.py:61-66: tensors over the same sites, summed."""
    from .tensor import SparseConvNetTensor
    total = input[0].features
    for i in input[1:]:
        total = total + i.features
    return SparseConvNetTensor(total, input[0].metadata, input[0].spatial_size)


def append_tensors(tensors):
    """utils.py:68-77 over Metadata::appendMetadata (Metadata/Metadata.cpp:248-262): the samples
    of every tensor after those of the ones before it, rows in the same order.  The new
    Metadata is built from the tensors' site lists (mode 0: rows = points)."""
    from .metadata import Metadata
    from .tensor import SparseConvNetTensor
    spatial_size = tensors[0].spatial_size
    dimension = len(spatial_size)
    locations, first_sample = [], 0
    for t in tensors:
        loc = t.get_spatial_locations().clone()
        loc[:, -1] += first_sample
        locations.append(loc)
        first_sample += t.batch_size()
    features = torch.cat([t.features for t in tensors], 0)
    md = Metadata(dimension)
    rows = md.inputLayer(spatial_size, torch.cat(locations), features, first_sample, 0)
    return SparseConvNetTensor(rows, md, spatial_size)


class AddCoords(torch.nn.Module):
    """utils.py:79-92: appends every site's coordinates, scaled to [-1, 1], as extra planes."""

    def forward(self, input):
        from .tensor import SparseConvNetTensor
        features = input.features
        if features.numel():
            with torch.no_grad():
                coords = input.get_spatial_locations()[:, :-1].to(features)
                half = (input.spatial_size.to(features) - 1) / 2
                coords = coords / half[None, :] - 1
            features = torch.cat([features, coords], 1)
        return SparseConvNetTensor(features, input.metadata, input.spatial_size)

    def input_spatial_size(self, out_size):
        return out_size


def compare_sparse(x, y):
    """utils.py:94-108 over Metadata::compareSparseHelper (Metadata/Metadata.cpp:585-616): mean
    over the union of the two tensors' sites of the squared feature difference, a site missing
    on one side counting with its squared features."""
    dev = x.features.device
    lx, ly = x.get_spatial_locations().to(dev), y.get_spatial_locations().to(dev)
    both = torch.cat([lx, ly])
    _, site = torch.unique(both, dim=0, return_inverse=True)
    n = int(site.max()) + 1 if site.numel() else 0
    planes = max(x.features.size(1) if x.features.dim() == 2 else 0, y.features.size(1) if y.features.dim() == 2 else 0)
    diff = torch.zeros((n, planes), dtype=x.features.dtype, device=dev)
    if lx.size(0):
        diff.index_add_(0, site[:lx.size(0)], x.features)
    if ly.size(0):
        diff.index_add_(0, site[lx.size(0):], -y.features)
    return diff.pow(2).sum() / n
