"""The modules of the path, with the constructor signatures, attribute names, parameter
shapes, initialisation, spatial-size arithmetic and repr of the reference's Python modules
(cited per class; paths relative to the reference's sparseconvnet/ directory).  Each forward
and each backward calls the HIP library through sparseconvnet_amd.metadata; the
torch.autograd.Function classes mirror the reference's *Function classes."""
import torch
from torch.autograd import Function
from torch.nn import Module, Parameter

import sparseconvnet_amd as _pkg

from . import metadata as _md
from .tensor import SparseConvNetTensor
from .utils import optionalTensor, toLongTensor


def _opt(t):
    """None for the empty tensor that stands for "no bias" (utils.py:21-22)."""
    return t if t is not None and t.numel() else None


class _FrozenParams:
    """What a convolution module keeps between eval-mode calls: a scn_params object of the library
    (packed weights, folded batch norms) and the state of the tensors it was derived from.  The
    state is (address, version counter) per tensor: optimiser steps, load_state_dict, .cuda() and
    every other in-place write or replacement change it, and the object is cleared.  Writes
    through `tensor.data` do not move the version counter: after such a write in eval mode call
    sparseconvnet_amd.parameters_changed(), or switch sparseconvnet_amd.frozen_parameters off."""

    def __init__(self):
        self.handle, self.state, self.epoch = None, None, -1

    def use(self, md, tensors):
        if not _pkg.frozen_parameters:
            return
        L = _md._lib.lib()
        state = tuple((t.data_ptr(), t._version) for t in tensors if t is not None)
        if self.handle is None:
            self.handle = L.scn_params_create()
        if state != self.state or self.epoch != _pkg._parameter_epoch:
            _md._lib.check(L.scn_params_clear(self.handle))
            self.state, self.epoch = state, _pkg._parameter_epoch
        _md._lib.check(L.scn_md_use_params(md._h, self.handle))

    def __deepcopy__(self, memo):  # a copied or unpickled module starts with nothing kept
        return _FrozenParams()

    def __reduce__(self):
        return (_FrozenParams, ())

    def __del__(self):
        try:
            if self.handle is not None:
                _md._lib.lib().scn_params_destroy(self.handle)
        except Exception:
            pass


def _use_frozen(module, md, weight, bias, pre=None, post=None, second=None):
    """Eval mode: the module's convolution may keep what it derives from its parameters."""
    if module.training:
        return
    f = module.__dict__.get('_frozen')
    if f is None:
        f = module.__dict__['_frozen'] = _FrozenParams()
    tensors = [weight, bias]
    for bn in (pre, post, second[0] if second is not None else None):
        if bn is not None:
            tensors += list(bn[:4])
    f.use(md, tensors)


class _NoGrad:
    """What a Function's forward is handed in place of its context when nothing will be
    differentiated: attributes can be set on it, saved tensors are dropped."""

    def save_for_backward(self, *tensors):
        pass


def _call(fn, *args):
    """fn.apply(*args); with gradients disabled (inference under torch.no_grad()) the forward is
    called directly: Function.apply costs several microseconds per module call there, for an
    output that would carry no history either way."""
    if torch.is_grad_enabled():
        return fn.apply(*args)
    return fn.forward(_NoGrad(), *args)


class _ConvFunction(Function):
    """submanifoldConvolution.py:63-113, convolution.py:72-130, deconvolution.py:49-128: kind 0 /
    1 / 2.  pre / post: eval-mode batch norms applied inside the convolution (inference only)."""

    @staticmethod
    def forward(ctx, features, weight, bias, md, kind, sizes, pre, post, out=None, second=None):
        ctx.md, ctx.kind, ctx.sizes, ctx.fused = md, kind, sizes, pre is not None or post is not None
        ctx.has_bias = bias.numel() > 0
        ctx.save_for_backward(features, weight)
        fn = (md.submanifoldConvolution, md.convolution, md.deconvolution)[kind]
        out, _ = fn(*sizes, features, weight, bias, pre, post, want_macs=False, out=out, second=second)
        _count(out)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        # batchNormalization.py:147: the reference refuses to differentiate an eval-mode batch norm
        assert not ctx.fused, "backward through an eval-mode batch normalisation; call .train() on the model"
        features, weight = ctx.saved_tensors
        fn = (ctx.md.submanifoldConvolutionBackward, ctx.md.convolutionBackward, ctx.md.deconvolutionBackward)[ctx.kind]
        d_in, d_w, d_b = fn(*ctx.sizes, features, grad_output.contiguous(), weight, ctx.has_bias)
        return d_in, d_w, d_b, None, None, None, None, None, None, None


class _NetworkInNetworkFunction(Function):
    """networkInNetwork.py:13-56."""

    @staticmethod
    def forward(ctx, features, weight, bias, md):
        ctx.md, ctx.has_bias = md, bias.numel() > 0
        ctx.save_for_backward(features, weight)
        out, _ = md.networkInNetwork(features, weight, bias, want_macs=False)
        _count(out)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        features, weight = ctx.saved_tensors
        d_in, d_w, d_b = ctx.md.networkInNetworkBackward(features, grad_output.contiguous(), weight, ctx.has_bias)
        return d_in, d_w, d_b, None


class _BatchNormalizationFunction(Function):
    """batchNormalization.py:93-160."""

    @staticmethod
    def forward(ctx, features, weight, bias, running_mean, running_var, eps, momentum, train, leakiness, md):
        ctx.md, ctx.train, ctx.leakiness, ctx.affine = md, train, leakiness, weight.numel() > 0
        if train:
            out, save_mean, save_invstd = md.batchNormTrain(features, running_mean, running_var, _opt(weight),
                                                            _opt(bias), eps, momentum, leakiness)
            ctx.save_for_backward(features, out, weight, save_mean, save_invstd)
        else:
            out = _md.batchNormEval(features, running_mean, running_var, _opt(weight), _opt(bias), eps, leakiness)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        assert ctx.train, "backward through an eval-mode batch normalisation; call .train() on the model"
        features, out, weight, save_mean, save_invstd = ctx.saved_tensors
        d_in, d_w, d_b = ctx.md.batchNormBackward(features, out, grad_output.contiguous(), save_mean, save_invstd,
                                                  _opt(weight), ctx.leakiness, ctx.affine)
        return d_in, d_w, d_b, None, None, None, None, None, None, None


class _JoinBatchNormFunction(Function):
    """JoinTable followed by an eval-mode batch normalisation (tables.py:35-48,
    batchNormalization.py:93-117) in one pass per part: each part is normalised with its range
    of the planes straight into its columns of the joined matrix, which costs what the
    concatenation alone costs and spares the convolution behind it the normalisation."""

    @staticmethod
    def forward(ctx, running_mean, running_var, weight, bias, eps, leakiness, *parts):
        rows = parts[0].size(0)
        out = parts[0].new_empty((rows, sum(p.size(1) for p in parts)))
        off = 0
        for p in parts:
            c = p.size(1)
            _md.batchNormEval(p, running_mean[off:off + c], running_var[off:off + c],
                              weight[off:off + c] if weight.numel() else None,
                              bias[off:off + c] if bias.numel() else None, eps, leakiness, out=out[:, off:off + c])
            off += c
        return out

    @staticmethod
    def backward(ctx, grad_output):
        # batchNormalization.py:147
        assert False, "backward through an eval-mode batch normalisation; call .train() on the model"


def join_batchnorm(parts, bn):
    """JoinTable()(parts) followed by the eval-mode batch normalisation `bn`, or None when the
    two have to run one after the other (plane counts that do not add up, empty tensors)."""
    if not _pkg.fuse_batchnorm or not _is_bn(bn) or len(parts) < 2:
        return None
    feats = [p.features for p in parts]
    if any(f.dim() != 2 or f.nelement() == 0 or f.size(0) != feats[0].size(0) for f in feats):
        return None
    if sum(f.size(1) for f in feats) != bn.nPlanes:
        return None
    output = SparseConvNetTensor()
    output.metadata = parts[0].metadata
    output.spatial_size = parts[0].spatial_size
    output.features = _call(_JoinBatchNormFunction, bn.running_mean, bn.running_var, optionalTensor(bn, 'weight').detach(),
                                                   optionalTensor(bn, 'bias').detach(), bn.eps, bn.leakiness, *feats)
    return output


def _bn_slice(bn, lo, hi):
    """The arguments _bn_args gives, for planes [lo, hi) of the batch normalisation."""
    w, b = optionalTensor(bn, 'weight').detach(), optionalTensor(bn, 'bias').detach()
    return (bn.running_mean[lo:hi], bn.running_var[lo:hi], w[lo:hi] if w.numel() else w, b[lo:hi] if b.numel() else b,
            bn.eps, bn.leakiness)


def skip_join_plan(conv, mods, input):
    """For a SubmanifoldConvolution `conv` about to run on `input` with `mods` behind it: when those
    begin with [ConcatTable(Identity, Sequential(... convolution)), JoinTable, eval-mode batch norm]
    (the skip connection of a U-Net level) and concat_join_batchnorm will take them, returns
    (batch norm, planes of the skip part): `conv` can then write the skip part of the joined matrix
    itself, normalised, beside its plain output (the `second` output of the convolutions)."""
    from .containers import ConcatTable, JoinTable, Sequential
    if not _pkg.fuse_batchnorm or torch.is_grad_enabled() or len(mods) < 3 or input.features.nelement() == 0:
        return None
    table, join, bn = mods[0], mods[1], mods[2]
    if type(conv) not in (SubmanifoldConvolution, ValidConvolution) or conv.groups != 1 or conv.nOut > 256:
        return None
    if type(table) is not ConcatTable or type(join) is not JoinTable or not _is_bn(bn):
        return None
    if any(m._forward_hooks or m._forward_pre_hooks for m in (table, join)):
        return None
    children = list(table._modules.values())
    if len(children) != 2 or not _plain(children[0], (Identity,)):
        return None
    last = children[1]
    if type(last) is not Sequential or last._forward_hooks or last._forward_pre_hooks:
        return None
    chain = last._chain()
    if not chain or not _is_conv(chain[-1]) or chain[-1].nOut > 256 or conv.nOut + chain[-1].nOut != bn.nPlanes:
        return None
    return bn, conv.nOut


def concat_join_batchnorm(table, bn, input, prefilled=None):
    """ConcatTable `table`, JoinTable and the eval-mode batch normalisation `bn` run on `input` with
    no pass over the joined matrix: when the table's last branch ends in a convolution (the
    Deconvolution of a U-Net level), that convolution applies its planes' share of the batch norm
    to its output and writes it straight into its columns of the joined matrix; the other
    branches' results are normalised into theirs as join_batchnorm does.  None when this does not
    apply (the caller then runs the three modules one after the other).  Inference only.
    prefilled: the joined matrix with the first branch's columns already written (skip_join_plan:
    that branch is the Identity and the producer of `input` wrote them)."""
    from .containers import Sequential
    if not _pkg.fuse_batchnorm or torch.is_grad_enabled() or not _is_bn(bn) or not isinstance(input, SparseConvNetTensor):
        return None
    children = list(table._modules.values())
    if len(children) < 2 or input.features.nelement() == 0:
        return None
    last = children[-1]
    if type(last) is not Sequential or last._forward_hooks or last._forward_pre_hooks:
        return None
    chain = last._chain()
    if not chain or not _is_conv(chain[-1]) or chain[-1].nOut > 256:
        return None
    conv = chain[-1]
    parts = [input] if prefilled is not None else [c(input) for c in children[:-1]]
    feats = [p.features for p in parts]
    rows = feats[0].size(0) if feats[0].dim() == 2 else -1
    fits = all(f.dim() == 2 and f.size(0) == rows and f.nelement() for f in feats) and \
        sum(f.size(1) for f in feats) + conv.nOut == bn.nPlanes
    if not fits:  # as the modules by themselves would
        parts.append(last(input))
        from .containers import JoinTable
        return bn(JoinTable()(parts))
    out = prefilled if prefilled is not None else feats[0].new_empty((rows, bn.nPlanes))
    off = 0
    for f in feats:
        c = f.size(1)
        if prefilled is None:
            mean, var, w, b, eps, leak = _bn_slice(bn, off, off + c)
            _md.batchNormEval(f, mean, var, _opt(w), _opt(b), eps, leak, out=out[:, off:off + c])
        off += c
    Sequential._run(chain, input, tail=(_bn_slice(bn, off, bn.nPlanes), out[:, off:]))
    output = SparseConvNetTensor()
    output.metadata = parts[0].metadata
    output.spatial_size = parts[0].spatial_size
    output.features = out
    return output


class _ActivePoolingFunction(Function):
    """The calls pybind.cpp:34-43 binds (the reference's Python package has no module over them)."""

    @staticmethod
    def forward(ctx, features, md, spatial_size, average):
        ctx.md, ctx.spatial_size, ctx.average, ctx.shape = md, spatial_size, average, tuple(features.shape)
        return md.activePooling(spatial_size, features, average)

    @staticmethod
    def backward(ctx, grad_output):
        return ctx.md.activePoolingBackward(ctx.spatial_size, ctx.shape, grad_output.contiguous(), ctx.average), \
            None, None, None


class _PoolingFunction(Function):
    """maxPooling.py:14-72, averagePooling.py:13-66, unPooling.py:14-57: which = 'max', 'average',
    'un'.  sizes = (input level, output level, pool size, pool stride) of the op."""

    @staticmethod
    def forward(ctx, features, md, which, sizes, drop):
        ctx.md, ctx.which, ctx.sizes, ctx.drop, ctx.shape = md, which, sizes, drop, tuple(features.shape)
        fn = {"max": md.maxPooling, "average": md.averagePooling, "un": md.unPooling}[which]
        out = fn(*sizes, features, drop)
        if which == "max":
            ctx.save_for_backward(features, out)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        g = grad_output.contiguous()
        if ctx.which == "max":
            features, out = ctx.saved_tensors
            d_in = ctx.md.maxPoolingBackward(*ctx.sizes, features, out, g, ctx.drop)
        elif ctx.which == "average":
            d_in = ctx.md.averagePoolingBackward(*ctx.sizes, ctx.shape, g, ctx.drop)
        else:
            d_in = ctx.md.unPoolingBackward(*ctx.sizes, ctx.shape, g, ctx.drop)
        return d_in, None, None, None, None


class _InputLayerFunction(Function):
    """ioLayers.py:163-196 and :216-248 (bl)."""

    @staticmethod
    def forward(ctx, features, md, spatial_size, coords, batch_size, mode, bl):
        ctx.md, ctx.bl = md, bl
        if bl:
            return md.blInputLayer(spatial_size, coords, features, mode)
        return md.inputLayer(spatial_size, coords, features, batch_size, mode)

    @staticmethod
    def backward(ctx, grad_output):
        return ctx.md.inputLayerBackward(grad_output.contiguous(), ctx.bl), None, None, None, None, None, None


class _OutputLayerFunction(Function):
    """ioLayers.py:198-213 and :250-283 (bl)."""

    @staticmethod
    def forward(ctx, features, md, bl):
        ctx.md, ctx.rows = md, features.size(0)
        return md.blOutputLayer(features) if bl else md.outputLayer(features)

    @staticmethod
    def backward(ctx, grad_output):
        return ctx.md.outputLayerBackward(grad_output.contiguous(), ctx.rows), None, None


class _SparseToDenseFunction(Function):
    """sparseToDense.py:25-54."""

    @staticmethod
    def forward(ctx, features, md, spatial_size, planes):
        ctx.md, ctx.spatial_size, ctx.rows = md, spatial_size, features.size(0)
        return md.sparseToDense(spatial_size, features, planes)

    @staticmethod
    def backward(ctx, grad_output):
        return ctx.md.sparseToDenseBackward(ctx.spatial_size, grad_output.contiguous(), ctx.rows), None, None, None


def _size_repr(prefix, size, stride=None):
    """'C3', 'C(3,1,3)', 'C3/2', 'C(3,3)/(2,1)' ... as the reference prints filter sizes."""
    uniform = size.max().item() == size.min().item() and (
        stride is None or stride.max().item() == stride.min().item())
    if uniform:
        s = prefix + str(size[0].item())
        if stride is not None:
            s += '/' + str(stride[0].item())
        return s
    s = prefix + '(' + ','.join(str(v.item()) for v in size) + ')'
    if stride is not None:
        s += '/(' + ','.join(str(v.item()) for v in stride) + ')'
    return s


def _conv_weight(filter_volume, groups, nIn, nOut):
    # N(0, sqrt(2 * groups / (nIn * filter_volume))): submanifoldConvolution.py:23-26
    std = (2.0 * groups / nIn / filter_volume) ** 0.5
    return Parameter(torch.Tensor(filter_volume, groups, nIn // groups, nOut // groups).normal_(0, std))


def _count(out):
    # the multiply-adds are counted by the library (Metadata.takeMacs), see metadata.MacCounter
    _pkg.forward_pass_hidden_states += out.nelement()


def _bn_args(bn):
    """The tensors and constants of an eval-mode BatchNormalization module that a convolution
    applies to its input rows itself (None: nothing to apply)."""
    if bn is None or isinstance(bn, tuple):
        return bn
    return (bn.running_mean, bn.running_var, optionalTensor(bn, 'weight').detach(),
            optionalTensor(bn, 'bias').detach(), bn.eps, bn.leakiness)


def _plain(module, classes):
    return type(module) in classes and not module._forward_hooks and not module._forward_pre_hooks


def _is_bn(module):
    return (_plain(module, (BatchNormalization, BatchNormReLU, BatchNormLeakyReLU)) and not module.training)


def _is_conv(module):
    return (_plain(module, (SubmanifoldConvolution, ValidConvolution, Convolution, Deconvolution))
            and module.groups == 1)


def fuse_plan(mods, input):
    """How Sequential runs the first module(s) of `mods` on `input`: (convolution, batch norm in
    front or None, batch norm behind or None, number of modules consumed), or None when the
    first module runs by itself.  An eval-mode batch normalisation next to a convolution gives
    the same result applied inside the convolution, without a pass over the rows of its own."""
    if not _pkg.fuse_batchnorm or input.features.nelement() == 0:
        return None
    pre, i = None, 0
    if len(mods) > 1 and _is_bn(mods[0]) and _is_conv(mods[1]) and mods[0].nPlanes == mods[1].nIn:
        pre, i = mods[0], 1
    if not _is_conv(mods[i]) or input.features.size(1) != mods[i].nIn:
        return None
    conv = mods[i]
    post = None
    if len(mods) > i + 1 and _is_bn(mods[i + 1]) and mods[i + 1].nPlanes == conv.nOut:
        post = mods[i + 1]
    if pre is None and post is None:
        return None
    return conv, pre, post, i + 1 + (post is not None)


class SubmanifoldConvolution(Module):
    """submanifoldConvolution.py:14-61."""

    def __init__(self, dimension, nIn, nOut, filter_size, bias, groups=1):
        Module.__init__(self)
        self.dimension = dimension
        self.groups = groups
        self.nIn = nIn
        self.nOut = nOut
        self.filter_size = toLongTensor(dimension, filter_size)
        self.filter_volume = self.filter_size.prod().item()
        self.weight = _conv_weight(self.filter_volume, groups, nIn, nOut)
        if bias:
            self.bias = Parameter(torch.Tensor(nOut).zero_())

    def forward(self, input, pre_bn=None, post_bn=None, out=None, second=None):
        assert input.features.nelement() == 0 or input.features.size(1) == self.nIn, (self.nIn, self.nOut, input)
        output = SparseConvNetTensor()
        output.metadata = input.metadata
        output.spatial_size = input.spatial_size
        pre, post = _bn_args(pre_bn), _bn_args(post_bn)
        _use_frozen(self, input.metadata, self.weight, optionalTensor(self, 'bias'), pre, post, second)
        output.features = _call(_ConvFunction, input.features, self.weight, optionalTensor(self, 'bias'), input.metadata, 0,
                                              (input.spatial_size, self.filter_size), pre, post, out, second)
        return output

    def __repr__(self):
        return 'SubmanifoldConvolution ' + str(self.nIn) + '->' + str(self.nOut) + _size_repr(' C', self.filter_size)

    def input_spatial_size(self, out_size):
        return out_size


class ValidConvolution(SubmanifoldConvolution):
    pass


class Convolution(Module):
    """convolution.py:13-70."""

    def __init__(self, dimension, nIn, nOut, filter_size, filter_stride, bias, groups=1):
        Module.__init__(self)
        self.dimension = dimension
        self.groups = groups
        self.nIn = nIn
        self.nOut = nOut
        self.filter_size = toLongTensor(dimension, filter_size)
        self.filter_volume = self.filter_size.prod().item()
        self.filter_stride = toLongTensor(dimension, filter_stride)
        self.weight = _conv_weight(self.filter_volume, groups, nIn, nOut)
        if bias:
            self.bias = Parameter(torch.Tensor(nOut).zero_())

    def forward(self, input, pre_bn=None, post_bn=None, out=None, second=None):
        assert input.features.nelement() == 0 or input.features.size(1) == self.nIn
        output = SparseConvNetTensor()
        output.metadata = input.metadata
        output.spatial_size = (input.spatial_size - self.filter_size).div(
            self.filter_stride, rounding_mode='trunc') + 1
        assert ((output.spatial_size - 1) * self.filter_stride + self.filter_size == input.spatial_size).all(), (
            input.spatial_size, output.spatial_size, self.filter_size, self.filter_stride)
        a = (input.spatial_size, output.spatial_size, self.filter_size, self.filter_stride)
        pre, post = _bn_args(pre_bn), _bn_args(post_bn)
        _use_frozen(self, input.metadata, self.weight, optionalTensor(self, 'bias'), pre, post, second)
        output.features = _call(_ConvFunction, input.features, self.weight, optionalTensor(self, 'bias'), input.metadata, 1,
                                              a, pre, post, out, second)
        return output

    def __repr__(self):
        return 'Convolution ' + str(self.nIn) + '->' + str(self.nOut) + _size_repr(
            ' C', self.filter_size, self.filter_stride)

    def input_spatial_size(self, out_size):
        return (out_size - 1) * self.filter_stride + self.filter_size


class Deconvolution(Module):
    """deconvolution.py:13-47,76-100: undoes the matching Convolution's change of level."""

    def __init__(self, dimension, nIn, nOut, filter_size, filter_stride, bias, groups=1):
        Module.__init__(self)
        self.dimension = dimension
        self.groups = groups
        self.nIn = nIn
        self.nOut = nOut
        self.filter_size = toLongTensor(dimension, filter_size)
        self.filter_volume = self.filter_size.prod().item()
        self.filter_stride = toLongTensor(dimension, filter_stride)
        self.weight = _conv_weight(self.filter_volume, groups, nIn, nOut)
        if bias:
            self.bias = Parameter(torch.Tensor(nOut).zero_())

    def forward(self, input, pre_bn=None, post_bn=None, out=None, second=None):
        assert input.features.nelement() == 0 or input.features.size(1) == self.nIn
        output = SparseConvNetTensor()
        output.metadata = input.metadata
        output.spatial_size = (input.spatial_size - 1) * self.filter_stride + self.filter_size
        a = (input.spatial_size, output.spatial_size, self.filter_size, self.filter_stride)
        pre, post = _bn_args(pre_bn), _bn_args(post_bn)
        _use_frozen(self, input.metadata, self.weight, optionalTensor(self, 'bias'), pre, post, second)
        output.features = _call(_ConvFunction, input.features, self.weight, optionalTensor(self, 'bias'), input.metadata, 2,
                                              a, pre, post, out, second)
        return output

    def __repr__(self):
        return 'Deconvolution ' + str(self.nIn) + '->' + str(self.nOut) + _size_repr(
            ' C', self.filter_size, self.filter_stride)

    def input_spatial_size(self, out_size):
        in_size = (out_size - self.filter_size) / self.filter_stride + 1
        assert ((in_size - 1) * self.filter_stride + self.filter_size == out_size).all()
        return in_size


class NetworkInNetwork(Module):
    """networkInNetwork.py:57-93: a 1x1 convolution, out = bias + in @ weight."""

    def __init__(self, nIn, nOut, bias):
        Module.__init__(self)
        self.nIn = nIn
        self.nOut = nOut
        std = (2.0 / nIn)**0.5
        self.weight = Parameter(torch.Tensor(nIn, nOut).normal_(0, std))
        if bias:
            self.bias = Parameter(torch.Tensor(nOut).zero_())

    def forward(self, input):
        assert input.features.nelement() == 0 or input.features.size(1) == self.nIn, \
            (self.nIn, input.features.shape)
        output = SparseConvNetTensor()
        output.metadata = input.metadata
        output.spatial_size = input.spatial_size
        _use_frozen(self, input.metadata, self.weight, optionalTensor(self, 'bias'))
        output.features = _call(_NetworkInNetworkFunction, input.features, self.weight, optionalTensor(self, 'bias'),
                                                          input.metadata)
        return output

    def __repr__(self):
        return 'NetworkInNetwork' + str(self.nIn) + '->' + str(self.nOut)

    def input_spatial_size(self, out_size):
        return out_size


class BatchNormalization(Module):
    """batchNormalization.py:13-71.  leakiness: 0 = ReLU, (0,1) = leaky ReLU, 1 = none.
    Training mode normalises with the batch statistics and updates the running ones
    (momentum weights the old value); eval mode uses the running statistics as they are."""

    def __init__(self, nPlanes, eps=1e-4, momentum=0.99, affine=True, leakiness=1):
        Module.__init__(self)
        self.nPlanes = nPlanes
        self.eps = eps
        self.momentum = momentum
        self.affine = affine
        self.leakiness = leakiness
        self.register_buffer("running_mean", torch.Tensor(nPlanes).fill_(0))
        self.register_buffer("running_var", torch.Tensor(nPlanes).fill_(1))
        if affine:
            self.weight = Parameter(torch.Tensor(nPlanes).fill_(1))
            self.bias = Parameter(torch.Tensor(nPlanes).fill_(0))

    def forward(self, input):
        if input.features.nelement() == 0:
            return input
        assert input.features.size(1) == self.nPlanes, (self.nPlanes, input.features.shape)
        output = SparseConvNetTensor()
        output.metadata = input.metadata
        output.spatial_size = input.spatial_size
        output.features = _call(_BatchNormalizationFunction,
            input.features, optionalTensor(self, 'weight'), optionalTensor(self, 'bias'), self.running_mean,
            self.running_var, self.eps, self.momentum, self.training, self.leakiness, input.metadata)
        return output

    def input_spatial_size(self, out_size):
        return out_size

    def __repr__(self):
        s = 'BatchNorm(' + str(self.nPlanes) + ',eps=' + str(self.eps) + ',momentum=' + str(self.momentum) + \
            ',affine=' + str(self.affine)
        if self.leakiness > 0:
            s = s + ',leakiness=' + str(self.leakiness)
        return s + ')'


class BatchNormReLU(BatchNormalization):
    """batchNormalization.py:74-81."""

    def __init__(self, nPlanes, eps=1e-4, momentum=0.99):
        BatchNormalization.__init__(self, nPlanes, eps, momentum, True, 0)

    def __repr__(self):
        return 'BatchNormReLU(' + str(self.nPlanes) + ',eps=' + str(self.eps) + ',momentum=' + \
            str(self.momentum) + ',affine=' + str(self.affine) + ')'


class BatchNormLeakyReLU(BatchNormalization):
    """batchNormalization.py:84-91."""

    def __init__(self, nPlanes, eps=1e-4, momentum=0.99, leakiness=0.333):
        BatchNormalization.__init__(self, nPlanes, eps, momentum, True, leakiness)

    def __repr__(self):
        return 'BatchNormLeakyReLU(' + str(self.nPlanes) + ',eps=' + str(self.eps) + ',momentum=' + \
            str(self.momentum) + ',affine=' + str(self.affine) + ',leakiness=' + str(self.leakiness) + ')'


class MaxPooling(Module):
    """maxPooling.py:74-117."""

    def __init__(self, dimension, pool_size, pool_stride, nFeaturesToDrop=0):
        super(MaxPooling, self).__init__()
        self.dimension = dimension
        self.pool_size = toLongTensor(dimension, pool_size)
        self.pool_stride = toLongTensor(dimension, pool_stride)
        self.nFeaturesToDrop = nFeaturesToDrop

    def forward(self, input):
        output = SparseConvNetTensor()
        output.metadata = input.metadata
        output.spatial_size = (input.spatial_size - self.pool_size).div(
            self.pool_stride, rounding_mode='trunc') + 1
        assert ((output.spatial_size - 1) * self.pool_stride + self.pool_size == input.spatial_size).all()
        a = (input.spatial_size, output.spatial_size, self.pool_size, self.pool_stride)
        output.features = _call(_PoolingFunction, input.features, input.metadata, "max", a, self.nFeaturesToDrop)
        return output

    def input_spatial_size(self, out_size):
        return (out_size - 1) * self.pool_stride + self.pool_size

    def __repr__(self):
        s = _size_repr('MaxPooling', self.pool_size, self.pool_stride)
        if self.nFeaturesToDrop > 0:
            s = s + ' nFeaturesToDrop = ' + str(self.nFeaturesToDrop)
        return s


class AveragePooling(MaxPooling):
    """averagePooling.py:13-67: the sum of the window's active inputs over the filter volume."""

    def forward(self, input):
        output = SparseConvNetTensor()
        output.metadata = input.metadata
        output.spatial_size = (input.spatial_size - self.pool_size).div(
            self.pool_stride, rounding_mode='trunc') + 1
        assert ((output.spatial_size - 1) * self.pool_stride + self.pool_size == input.spatial_size).all()
        a = (input.spatial_size, output.spatial_size, self.pool_size, self.pool_stride)
        output.features = _call(_PoolingFunction, input.features, input.metadata, "average", a, self.nFeaturesToDrop)
        return output

    def __repr__(self):
        return 'Average' + MaxPooling.__repr__(self)[3:]


class UnPooling(Module):
    """unPooling.py:59-96: every site of the finer level (which must exist in the metadata
    already) receives the rows of the coarse sites whose pooling windows hold it."""

    def __init__(self, dimension, pool_size, pool_stride, nFeaturesToDrop=0):
        super(UnPooling, self).__init__()
        self.dimension = dimension
        self.pool_size = toLongTensor(dimension, pool_size)
        self.pool_stride = toLongTensor(dimension, pool_stride)
        self.nFeaturesToDrop = nFeaturesToDrop

    def forward(self, input):
        output = SparseConvNetTensor()
        output.metadata = input.metadata
        output.spatial_size = (input.spatial_size - 1) * self.pool_stride + self.pool_size
        a = (input.spatial_size, output.spatial_size, self.pool_size, self.pool_stride)
        output.features = _call(_PoolingFunction, input.features, input.metadata, "un", a, self.nFeaturesToDrop)
        return output

    def input_spatial_size(self, out_size):
        return (out_size - 1) * self.pool_stride + self.pool_size

    def __repr__(self):
        s = _size_repr('UnPooling', self.pool_size, self.pool_stride)
        if self.nFeaturesToDrop > 0:
            s = s + ' nFeaturesToDrop = ' + str(self.nFeaturesToDrop)
        return s


class InputLayer(Module):
    """ioLayers.py:15-65.  forward takes (coords, features[, batch_size]): coords is an int64
    tensor [N, dimension] (one sample) or [N, dimension+1] (last column = sample index),
    features a float tensor [N, planes].  Points that share a site are merged according to
    mode: 0 none (rows = points), 1 first, 2 last, 3 sum, 4 mean - as the reference's rule
    builder behaves (Metadata/IOLayersRules.h:96-107), not as its docstring says for 1 and 2."""

    def __init__(self, dimension, spatial_size, mode=3):
        Module.__init__(self)
        self.dimension = dimension
        self.spatial_size = toLongTensor(dimension, spatial_size)
        self.mode = mode
        self.device = None

    def to(self, device):
        self.device = device
        return self

    def forward(self, input):
        output = SparseConvNetTensor(metadata=_md.Metadata(self.dimension), spatial_size=self.spatial_size)
        feats = input[1].to(self.device) if self.device else input[1]
        if not feats.is_cuda:
            feats = feats.cuda()
        batch_size = 0 if len(input) == 2 else input[2]
        output.features = _call(_InputLayerFunction, feats.float(), output.metadata, self.spatial_size, input[0], batch_size,
                                                    self.mode, False)
        return output


class OutputLayer(Module):
    """ioLayers.py:68-89: one row per original input point."""

    def __init__(self, dimension):
        Module.__init__(self)
        self.dimension = dimension

    def forward(self, input):
        return _call(_OutputLayerFunction, input.features, input.metadata, False)


class BLInputLayer(Module):
    """ioLayers.py:92-138.  forward takes (coords, features): coords an int64 tensor
    [batch, length, dimension] whose positions with a negative first coordinate are empty,
    features a float tensor [batch, length, planes].  mode 0: every position is a row;
    1: the last point of a site, 2: the first, 3: sum, 4: mean."""

    def __init__(self, dimension, spatial_size, mode=3):
        Module.__init__(self)
        self.dimension = dimension
        self.spatial_size = toLongTensor(dimension, spatial_size)
        self.mode = mode
        self.device = None

    def to(self, device):
        self.device = device
        return self

    def forward(self, input):
        output = SparseConvNetTensor(metadata=_md.Metadata(self.dimension), spatial_size=self.spatial_size)
        feats = input[1].to(self.device) if self.device else input[1]
        if not feats.is_cuda:
            feats = feats.cuda()
        output.features = _call(_InputLayerFunction, feats.float(), output.metadata, self.spatial_size, input[0], 0,
                                                    self.mode, True)
        return output


class BLOutputLayer(Module):
    """ioLayers.py:141-160: [batch, length, planes], zeros at the empty positions."""

    def __init__(self, dimension):
        Module.__init__(self)
        self.dimension = dimension

    def forward(self, input):
        return _call(_OutputLayerFunction, input.features, input.metadata, True)


class ActivePooling(Module):
    """Sums (average=True: averages) the active rows of every sample: a dense [batchSize, nPlanes]
    tensor, whatever the spatial size (SCN/CPU/ActivePooling.cpp:47-63, bound by pybind.cpp:34-43;
    sparseToDense.py:9 names it as the other way out of a sparse network.  The reference ships no
    Python class for it; the constructor follows its pooling modules)."""

    def __init__(self, dimension, average=False):
        Module.__init__(self)
        self.dimension = dimension
        self.average = average

    def forward(self, input):
        return _call(_ActivePoolingFunction, input.features, input.metadata, input.spatial_size, self.average)

    def input_spatial_size(self, out_size):
        return out_size

    def __repr__(self):
        return 'ActivePooling(average)' if self.average else 'ActivePooling'


class SparseToDense(Module):
    """sparseToDense.py:56-78: dense [batch, nPlanes, spatial...] tensor, zeros elsewhere."""

    def __init__(self, dimension, nPlanes):
        Module.__init__(self)
        self.dimension = dimension
        self.nPlanes = nPlanes

    def forward(self, input):
        return _call(_SparseToDenseFunction, input.features, input.metadata, input.spatial_size, self.nPlanes)

    def input_spatial_size(self, out_size):
        return out_size

    def __repr__(self):
        return 'SparseToDense(' + str(self.dimension) + ',' + str(self.nPlanes) + ')'


class Identity(Module):
    """identity.py:10-15."""

    def forward(self, input):
        return input

    def input_spatial_size(self, out_size):
        return out_size


class DenseToSparse(Module):
    """denseToSparse.py:13-67 over Metadata::createMetadataForDenseToSparse
    (Metadata/Metadata.cpp:177-214): a dense [batch, planes, spatial...] tensor becomes a
    sparse one whose sites are the cells with a non-zero plane, rows in (sample, row-major
    cell) order.  Here: the non-zero cells' coordinates go through the input-layer construction
    in mode 0 (rows = points)."""

    def __init__(self, dimension):
        Module.__init__(self)
        self.dimension = dimension

    def forward(self, input):
        d = self.dimension
        assert input.dim() == d + 2
        if not input.is_cuda:
            input = input.cuda()
        output = SparseConvNetTensor(metadata=_md.Metadata(d), spatial_size=torch.LongTensor(list(input.shape[2:])))
        cells = input.detach().permute(0, *range(2, 2 + d), 1)      # [batch, spatial..., planes]
        nz = (cells.abs().sum(-1) != 0).nonzero()                    # [n, 1 + d]: sample first
        coords = torch.cat([nz[:, 1:], nz[:, :1]], 1).contiguous()   # the library's column order
        md, sz, batch = output.metadata, output.spatial_size, input.size(0)

        def gather(x):
            rows = x.permute(0, *range(2, 2 + d), 1)[tuple(nz.t())].float().contiguous()
            return md.inputLayer(sz, coords, rows, batch, 0)
        with torch.no_grad():
            output.features = gather(input)
        return output

    def input_spatial_size(self, out_size):
        return out_size

    def __repr__(self):
        return 'DenseToSparse(' + str(self.dimension) + ')'


class InputLayerInput(object):
    """ioLayers.py:285-294: the (coords, features) pair an InputLayer takes, with .cuda()."""

    def __init__(self, coords, features):
        self.x = [coords, features]

    def __getitem__(self, n):
        return self.x[n]

    def __len__(self):
        return 2

    def cuda(self):
        self.x[1] = self.x[1].cuda()
        return self
