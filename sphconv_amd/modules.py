"""Containers (reference: sphconv/modules.py:36-132)."""
import sys
from collections import OrderedDict

import torch
from torch import nn


class SphModule(nn.Module):
    """Marker base class: modules derived from it receive the SparseConvTensor
    itself inside :class:`Sequential`; any other module receives ``.feature``."""


def is_sph_module(module) -> bool:
    return isinstance(module, SphModule)


def is_sparse_conv(module) -> bool:
    from .conv import Convolution
    return isinstance(module, Convolution)


def _bn_affine(bn: nn.BatchNorm1d):
    """Evaluation-mode BatchNorm1d as y = x*scale + shift (fp32 [C]); computed once per state of
    the module's tensors (their version counters) and kept on the module."""
    tensors = (bn.running_mean, bn.running_var, bn.weight, bn.bias)
    key = tuple((t.data_ptr(), t._version, t.dtype) if t is not None else None for t in tensors) + (bn.eps,)
    cached = getattr(bn, "_sph_affine", None)
    if cached is not None and cached[0] == key:
        return cached[1], cached[2]
    scale, shift = _bn_affine_now(bn)
    bn._sph_affine = (key, scale, shift)
    return scale, shift


def _bn_affine_now(bn: nn.BatchNorm1d):
    var = bn.running_var.float()
    scale = torch.rsqrt(var + bn.eps)
    if bn.weight is not None:
        scale = scale * bn.weight.float()
    shift = -bn.running_mean.float() * scale
    if bn.bias is not None:
        shift = shift + bn.bias.float()
    return scale.contiguous(), shift.contiguous()


class Sequential(SphModule):
    """Sequential container over sparse-conv and ordinary modules
    (modules.py:43-128).  Accepts positional modules, one OrderedDict, or keyword
    modules.

    With gradients disabled, a convolution followed by an evaluation-mode
    ``BatchNorm1d`` and/or a ``ReLU`` runs as one kernel: the affine map and the
    clamp are applied to the fp32 accumulators before the store (no reference
    counterpart: modules.py:124-125 runs them as separate passes over ``.feature``).
    ``fuse_eval = False`` switches this off."""

    fuse_eval = True
    # A strided convolution needs its output row count on the host before its rules can be generated.  The
    # container starts that count as soon as the layer's input coordinates exist -- at the container's input,
    # or behind the strided layer before it, submanifold layers in between change no coordinates -- so that
    # the host reads it while the convolutions in between keep the GPU busy (no reference counterpart:
    # rules.cu:461 waits where the layer runs).  False counts where the layer runs.
    count_ahead = True

    def __init__(self, *args, **kwargs):
        super().__init__()
        if len(args) == 1 and isinstance(args[0], OrderedDict):
            for key, module in args[0].items():
                self.add_module(key, module)
        else:
            for idx, module in enumerate(args):
                self.add_module(str(idx), module)
        for name, module in kwargs.items():
            if name in self._modules:
                raise ValueError("name exists.")
            self.add_module(name, module)

    def __getitem__(self, idx):
        if not (-len(self) <= idx < len(self)):
            raise IndexError("index {} is out of range".format(idx))
        if idx < 0:
            idx += len(self)
        return list(self._modules.values())[idx]

    def __len__(self):
        return len(self._modules)

    def add(self, module, name=None):
        if name is None:
            name = str(len(self._modules))
            if name in self._modules:
                raise KeyError("name exists")
        self.add_module(name, module)

    def _fusable_tail(self, mods, i):
        """(number of modules after mods[i] that fold into its store, BatchNorm1d or None, relu)."""
        conv = mods[i]
        if not (self.fuse_eval and is_sparse_conv(conv)) or torch.is_grad_enabled():
            return 0, None, False
        if conv.weight.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            return 0, None, False
        n, bn, relu = 0, None, False
        nxt = mods[i + 1] if i + 1 < len(mods) else None
        if (type(nxt) is nn.BatchNorm1d and not nxt.training and nxt.running_mean is not None
                and nxt.num_features == conv.out_channels):
            bn, n = nxt, 1
            nxt = mods[i + 2] if i + 2 < len(mods) else None
        if type(nxt) is nn.ReLU:
            relu, n = True, n + 1
        return n, bn, relu

    def forward(self, input):
        from .tensor import SparseConvTensor
        mods = list(self._modules.items())
        only = [m for _, m in mods]
        skip = 0
        ahead = {}      # index of a strided convolution -> its count on the way

        def start_count(first):
            """The next strided convolution at or behind module `first` that sees `input`'s coordinates."""
            if not (self.count_ahead and isinstance(input, SparseConvTensor)):
                return
            for j in range(first, len(only)):
                m = only[j]
                if is_sparse_conv(m) and not m.subm:
                    if hasattr(m, "count_ahead"):
                        h = m.count_ahead(input)
                        if h is not None:
                            ahead[j] = h
                    return
                if is_sph_module(m) and not is_sparse_conv(m):
                    return          # a module that may change the coordinates

        start_count(0)
        for i, (name, module) in enumerate(mods):
            if skip:
                skip -= 1
                continue
            if is_sph_module(module):
                assert isinstance(input, SparseConvTensor)
                with torch.autograd.profiler.record_function("sphconv:{}:{}".format(type(module).__name__, name)):
                    skip, bn, relu = self._fusable_tail(only, i)
                    kw = {"ahead": ahead.pop(i)} if i in ahead else {}
                    if skip:
                        scale, shift = _bn_affine(bn) if bn is not None else (None, None)
                        input = module(input, epilogue=(scale, shift, relu), **kw)
                    else:
                        input = module(input, **kw)
                    if is_sparse_conv(module) and not module.subm:
                        start_count(i + 1)      # new coordinates: the next strided layer can start counting
            elif isinstance(input, SparseConvTensor):
                input.feature = module(input.feature)
            else:
                input = module(input)
        return input


SparseSequential = Sequential
