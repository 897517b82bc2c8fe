"""Small helpers shared by the modules (same names and meaning as the reference's
sparseconvnet/utils.py:11-26)."""
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


def optionalTensor(module, name):
    """module.<name> if it exists, else an empty tensor (how the reference passes 'no bias')."""
    return getattr(module, name) if hasattr(module, name) else torch.Tensor()


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
