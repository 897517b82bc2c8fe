"""Containers: Sequential and the table modules (reference: sequential.py:10-35,
tables.py:13-55).  They only route SparseConvNetTensors; feature concatenation and addition
are plain torch ops on the GPU."""
import torch

from .tensor import SparseConvNetTensor


class Sequential(torch.nn.Sequential):
    def _chain(self):
        """The modules this container runs, with nested plain Sequentials (no hooks of their
        own) spliced in, so that a batch normalisation and a convolution that meet across the
        boundary of two blocks can still be run as one."""
        out = []
        for m in self._modules.values():
            if type(m) is Sequential and not m._forward_hooks and not m._forward_pre_hooks:
                out.extend(m._chain())
            else:
                out.append(m)
        return out

    def forward(self, input):
        return self._run(self._chain(), input)

    @staticmethod
    def _run(mods, input, tail=None):
        """Same chain as sequential.py:10-35, except that eval-mode batch normalisations next
        to a convolution are applied inside that convolution (layers.fuse_plan), one behind a
        JoinTable while the parts are joined (layers.join_batchnorm), and one behind a ConcatTable
        and a JoinTable by whatever produces each part (layers.concat_join_batchnorm).
        tail: (batch norm arguments, output columns) for the convolution that ends `mods`: it
        applies that batch norm to its output and writes it into those columns."""
        from .layers import fuse_plan, join_batchnorm, concat_join_batchnorm, skip_join_plan, _bn_slice, _is_conv
        i = 0
        while i < len(mods):
            if type(mods[i]) is JoinTable and i + 1 < len(mods) and isinstance(input, (list, tuple)) \
                    and not mods[i]._forward_hooks and not mods[i]._forward_pre_hooks:
                joined = join_batchnorm(input, mods[i + 1])
                if joined is not None:
                    input = joined
                    i += 2
                    continue
            if type(mods[i]) is ConcatTable and i + 2 < len(mods) and type(mods[i + 1]) is JoinTable \
                    and not any(m._forward_hooks or m._forward_pre_hooks for m in mods[i:i + 2]):
                joined = concat_join_batchnorm(mods[i], mods[i + 2], input)
                if joined is not None:
                    input = joined
                    i += 3
                    continue
            plan = fuse_plan(mods[i:i + 3], input) if isinstance(input, SparseConvNetTensor) else None
            # a convolution in front of a U-Net level's skip connection writes the skip part of the join itself
            if isinstance(input, SparseConvNetTensor) and (plan is not None or _is_conv(mods[i])):
                conv, pre, post, used = plan if plan is not None else (mods[i], None, None, 1)
                skip = skip_join_plan(conv, mods[i + used:i + used + 3], input) if post is None else None
                if skip is not None:
                    bn, c0 = skip
                    joined = input.features.new_empty((input.features.size(0), bn.nPlanes))
                    x = conv(input, pre_bn=pre, second=(_bn_slice(bn, 0, c0), joined[:, :c0]))
                    done = concat_join_batchnorm(mods[i + used], bn, x, prefilled=joined)
                    if done is not None:
                        input = done
                        i += used + 3
                    else:  # (not expected: skip_join_plan looked at the same things) as the modules by themselves
                        input = x
                        i += used
                    continue
            if plan is None:
                if tail is not None and i == len(mods) - 1:
                    input = mods[i](input, post_bn=tail[0], out=tail[1])
                else:
                    input = mods[i](input)
                i += 1
            else:
                conv, pre, post, used = plan
                if tail is not None and i + used == len(mods) and post is None:
                    input = conv(input, pre_bn=pre, post_bn=tail[0], out=tail[1])
                else:
                    input = conv(input, pre_bn=pre, post_bn=post)
                i += used
        return input

    def input_spatial_size(self, out_size):
        for m in reversed(self._modules):
            out_size = self._modules[m].input_spatial_size(out_size)
        return out_size

    def __add__(self, x):
        r = Sequential()
        for m in self:
            r.append(m)
        for m in x:
            r.append(m)
        return r

    def add(self, module):
        self._modules[str(len(self._modules))] = module
        return self

    def insert(self, index, module):
        for i in range(len(self._modules), index, -1):
            self._modules[str(i)] = self._modules[str(i - 1)]
        self._modules[str(index)] = module

    def append(self, module):
        self._modules[str(len(self._modules))] = module
        return self


class CheckpointedSequential(Sequential):
    """sequential.py:66-73 trades memory for recomputation in the backward pass
    (torch.utils.checkpoint over the module chain); here it runs as Sequential, keeping its
    activations: the reference's other name for the same function."""


class _Table(torch.nn.Sequential):
    def __init__(self, *args):
        torch.nn.Sequential.__init__(self, *args)

    def add(self, module):
        self._modules[str(len(self._modules))] = module
        return self


class ConcatTable(_Table):
    """Applies every child to the same input; returns the list of results."""

    def forward(self, input):
        return [module(input) for module in self._modules.values()]

    def input_spatial_size(self, out_size):
        return self._modules['0'].input_spatial_size(out_size)


class JoinTable(_Table):
    """Concatenates the feature planes of a list of tensors on one level."""

    def forward(self, input):
        output = SparseConvNetTensor()
        output.metadata = input[0].metadata
        output.spatial_size = input[0].spatial_size
        output.features = torch.cat([i.features for i in input], 1) if input[0].features.numel() \
            else input[0].features
        return output

    def input_spatial_size(self, out_size):
        return out_size


class AddTable(_Table):
    """Adds the features of a list of tensors on one level."""

    def forward(self, input):
        output = SparseConvNetTensor()
        output.metadata = input[0].metadata
        output.spatial_size = input[0].spatial_size
        features = input[0].features  # the reference's sum(...) starts from 0: one pass more
        for i in input[1:]:
            features = features + i.features
        output.features = features
        return output

    def input_spatial_size(self, out_size):
        return out_size
