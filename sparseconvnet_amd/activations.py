"""Pointwise modules on the feature matrix (reference: activations.py:16-83, dropout.py:13-52).
They are plain torch ops in the reference too; the sites are untouched."""
import torch
import torch.nn.functional as F
from torch.nn import Module

from .tensor import SparseConvNetTensor


class _Pointwise(Module):
    def fn(self, x):
        raise NotImplementedError

    def forward(self, input):
        return SparseConvNetTensor(self.fn(input.features), input.metadata, input.spatial_size)

    def input_spatial_size(self, out_size):
        return out_size


class Sigmoid(_Pointwise):
    def fn(self, x):
        return torch.sigmoid(x)


class Tanh(_Pointwise):
    def fn(self, x):
        return torch.tanh(x)


class ReLU(_Pointwise):
    def fn(self, x):
        return F.relu(x)


class LeakyReLU(_Pointwise):
    def __init__(self, leak=1 / 3):
        Module.__init__(self)
        self.leak = leak

    def fn(self, x):
        return F.leaky_relu(x, self.leak)


class ELU(_Pointwise):
    def fn(self, x):
        return F.elu(x)


class SELU(_Pointwise):
    def fn(self, x):
        return F.selu(x)


def BatchNormELU(nPlanes, eps=1e-4, momentum=0.9):
    import sparseconvnet_amd as scn
    return scn.Sequential().add(scn.BatchNormalization(nPlanes, eps, momentum)).add(ELU())


class Dropout(_Pointwise):
    """dropout.py:13-31: in eval mode the features are scaled by 1 - p; in training mode every
    element is kept with probability 1 - p (and not rescaled)."""

    def __init__(self, p=0.5):
        Module.__init__(self)
        self.p = p

    def _mask_shape(self, x):
        return x.shape

    def fn(self, x):
        if self.training:
            keep = torch.full(self._mask_shape(x), 1 - self.p, dtype=x.dtype, device=x.device)
            return x * torch.bernoulli(keep)
        return x * (1 - self.p)


class BatchwiseDropout(Dropout):
    """dropout.py:34-52: one keep / drop decision per plane for the whole batch."""

    def _mask_shape(self, x):
        return (1, x.shape[1])
