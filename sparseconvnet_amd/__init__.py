"""sparseconvnet_amd: the forward pass of submanifold sparse convolutional networks on
AMD MI355X, with the module API of facebookresearch/SparseConvNet (`import sparseconvnet_amd
as scn`).  The modules call hand-written gfx950 kernels in libscn_hip.so through its C ABI
(include/scn_hip.h); tensors are ordinary PyTorch-ROCm tensors."""

# Counters the reference keeps at package level (sparseconvnet/__init__.py:7-8): multiply-adds
# and output elements of the convolutions run so far.  forward_pass_multiplyAdd_count is a
# property of this module (see the end of the file): reading it collects the counts the
# library has been keeping on the GPU side.
forward_pass_hidden_states = 0
# Sequential hands an eval-mode batch normalisation that sits directly in front of a
# convolution to that convolution (one pass over the rows instead of two).  False: run
# every module as a pass of its own.
fuse_batchnorm = True
# Eval-mode convolution modules keep what they derive from their parameters (weights in the matrix
# instructions' operand order, folded batch norms) between calls, keyed on every parameter tensor's
# address and version counter.  parameters_changed() drops all of it (needed only after writes that
# bypass the version counter, i.e. through tensor.data).
frozen_parameters = True
_parameter_epoch = 0


def parameters_changed():
    global _parameter_epoch
    _parameter_epoch += 1

# True: every Metadata created from now on runs its wide convolutions (more than 32 output
# planes, or 128 and more input planes) with bf16 operands and fp32 accumulation.  The
# reference computes in fp32 throughout, which is also the default here.
bf16_mfma = False

from .activations import (ELU, SELU, BatchNormELU, BatchwiseDropout, Dropout, LeakyReLU, ReLU,  # noqa: E402
                          Sigmoid, Tanh)
from .containers import AddTable, CheckpointedSequential, ConcatTable, JoinTable, Sequential  # noqa: E402
from .layers import (ActivePooling, AveragePooling, BatchNormalization, BatchNormLeakyReLU, BatchNormReLU,  # noqa: E402
                     BLInputLayer, BLOutputLayer, Convolution, Deconvolution, DenseToSparse, Identity, InputLayer,
                     InputLayerInput, MaxPooling,
                     NetworkInNetwork, OutputLayer, SparseToDense, SubmanifoldConvolution, UnPooling,
                     ValidConvolution)
from .inputBatch import InputBatch  # noqa: E402
from .metadata import Metadata  # noqa: E402
from .networks import FullyConvolutionalNet, SparseResNet, SparseVggNet, UNet  # noqa: E402
from .tensor import SparseConvNetTensor  # noqa: E402
from .utils import (AddCoords, add_feature_planes, append_tensors, checkpoint_restore,  # noqa: E402
                    checkpoint_save, compare_sparse, concatenate_feature_planes, is_power2,
                    optionalTensor, prepare_BLInput, toLongTensor)


def is_hip_build():
    """True when libscn_hip.so is present and loadable (the reference's SCN.is_cuda_build)."""
    from . import _lib
    try:
        _lib.lib()
        return True
    except Exception:
        return False


import sys as _sys  # noqa: E402
import types as _types  # noqa: E402

from .metadata import mac_counter as _mac_counter  # noqa: E402


class _Package(_types.ModuleType):
    @property
    def forward_pass_multiplyAdd_count(self):
        return _mac_counter.read()

    @forward_pass_multiplyAdd_count.setter
    def forward_pass_multiplyAdd_count(self, value):
        _mac_counter.reset(value)


_sys.modules[__name__].__class__ = _Package
