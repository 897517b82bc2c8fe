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
