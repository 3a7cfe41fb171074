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


class Sequential(SphModule):
    """Sequential container over sparse-conv and ordinary modules
    (modules.py:43-128).  Accepts positional modules, one OrderedDict, or keyword
    modules."""

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

    def forward(self, input):
        from .tensor import SparseConvTensor
        for name, module in self._modules.items():
            if is_sph_module(module):
                assert isinstance(input, SparseConvTensor)
                with torch.autograd.profiler.record_function("sphconv:{}:{}".format(type(module).__name__, name)):
                    input = module(input)
            elif isinstance(input, SparseConvTensor):
                input.feature = module(input.feature)
            else:
                input = module(input)
        return input


SparseSequential = Sequential
