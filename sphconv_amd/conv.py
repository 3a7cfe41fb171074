"""Convolution modules with the reference's constructor arguments and forward
semantics (sphconv/conv.py:40-210)."""
import math
from typing import List, Optional

import torch
import torch.nn as nn

from . import sphconv_cuda as ext
from .functional import ConvFunction
from .modules import SphModule
from .rulebook import RuleBook
from .tensor import SparseConvTensor
from .utils import _calculate_fan_in_and_fan_out, _triple, kaiming_uniform_, out_spatial


def get_tile_grid_shape(out_spatial_shape_DWH: List[int], tile_size: List[int]) -> List[int]:
    """conv.py:32-38"""
    return [-(-out_spatial_shape_DWH[0] // tile_size[0]), -(-out_spatial_shape_DWH[1] // tile_size[1])]


class Convolution(SphModule):
    """Holds the weight ``[K0,K1,K2,iC,oC]`` (conv.py:43-72).  As in the reference,
    a bias parameter can be created but is not applied by ``forward``."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride, padding, dilation,
                 groups: int, tile_size: List[int], bias: bool, subm: bool, name: Optional[str],
                 indice_key: Optional[str] = None, **kwargs):
        super().__init__(**kwargs)
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = kernel_size
        self.stride = stride
        self.padding = padding
        self.dilation = dilation
        self.groups = groups
        self.tile_size = tile_size
        self.subm = subm
        self.indice_key = indice_key
        self.name = name
        self.rule_book: Optional[RuleBook] = None
        self.weight = nn.Parameter(torch.empty((*kernel_size, in_channels, out_channels)))
        if bias:
            self.bias = nn.Parameter(torch.empty(out_channels))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            fan_in, _ = _calculate_fan_in_and_fan_out(self.weight)
            bound = 1 / math.sqrt(fan_in)
            nn.init.uniform_(self.bias, -bound, bound)

    def invalidate_packed(self):
        """Forgets the fragment-ordered copy of the weight that forward passes in eval mode keep under
        ``torch.no_grad()``.  In-place updates that bump the weight's version counter (optimizer steps,
        ``load_state_dict``, ``weight.mul_()``) are followed without this; updates through ``weight.data`` are not."""
        ext.invalidate_packed(self.weight)

    @property
    def rule_size(self):
        """``rule_size [NTile,KV]`` of the last forward in the reference's format
        (the reference stores it eagerly, conv.py:179; here it is materialised on
        first access)."""
        if self.rule_book is None:
            return None
        return self.rule_book.padded(self.tile_size)[1]

    def extra_repr(self):
        s = "{in_channels}, {out_channels}, kernel_size={kernel_size}, stride={stride}"
        if tuple(self.padding) != (0,) * len(self.padding):
            s += ", padding={padding}"
        if tuple(self.dilation) != (1,) * len(self.dilation):
            s += ", dilation={dilation}"
        if self.groups != 1:
            s += ", groups={groups}"
        if self.bias is None:
            s += ", bias=False"
        if self.subm:
            s += ", subm={subm}"
        return s.format(**self.__dict__)


class Conv3d(Convolution):
    """3-D sparse convolution on range-voxel tensors (conv.py:99-193)."""

    def __init__(self, in_channels, out_channels, kernel_size=3, stride=1, padding=0, dilation=1,
                 groups=1, bias=False, subm=False, tile_size=[2, 2], indice_key=None, name=None,
                 **kwargs):
        assert groups == 1, "groups not supported yet"
        super().__init__(in_channels, out_channels, _triple(kernel_size), _triple(stride),
                         _triple(padding), _triple(dilation), groups, tile_size, bias, subm, name,
                         indice_key=indice_key, **kwargs)

    def count_ahead(self, input: SparseConvTensor):
        """For a strided layer whose rules are not cached: starts counting its output rows on ``input``'s
        coordinates (RuleBook.count_ahead).  Give the result to ``forward(..., ahead=)`` with a tensor of the
        same coordinates.  None when there is nothing to do ahead."""
        if self.subm or input.find_rule(self.indice_key) is not None or not input.z_ptr.is_cuda:
            return None
        in_shape = [input.D, input.W, input.H]
        out_shape = out_spatial(in_shape, self.kernel_size, self.stride, self.padding, self.dilation)
        return RuleBook.count_ahead(input.z_idx, input.z_ptr, input.B, in_shape, out_shape, self.kernel_size,
                                    self.stride, self.padding, self.dilation)

    def _rules(self, input: SparseConvTensor, out_shape, ahead=None, keep: bool = True, training: bool = True):
        """Rule book of this layer on ``input``, shared through ``rule_cache`` when an
        ``indice_key`` is set (conv.py:159-177).  A book that is not cached yet is returned unbuilt (for a strided
        layer with its output coordinates): ``rule_conv`` generates its pairs in the launch that convolves them
        where that is faster, and otherwise, like every later use, builds it; ``keep``: that launch also writes
        the book (later layers share it, or a backward pass follows)."""
        cached = input.find_rule(self.indice_key)
        if cached is not None:
            return cached
        in_shape = [input.D, input.W, input.H]
        row_cols = getattr(input, "row_cols", None)
        if self.subm:
            book = RuleBook.build_subm(input.z_idx, input.z_ptr, input.B, in_shape, self.kernel_size,
                                       self.padding, self.dilation, row_cols=row_cols, lazy=True)
        else:
            book = RuleBook.build(input.z_idx, input.z_ptr, input.B, in_shape, out_shape,
                                  self.kernel_size, self.stride, self.padding, self.dilation, ahead=ahead,
                                  row_cols=row_cols, lazy=True)
        book.keep = bool(keep)
        if not training:
            book.forward_only = (self.in_channels, self.out_channels, input.feature.element_size())
        entry = (book.oz_idx, book.oz_ptr, book, None, get_tile_grid_shape(out_shape, self.tile_size))
        if self.indice_key is not None:
            input.rule_cache[self.indice_key] = entry
        return entry

    def forward(self, input: SparseConvTensor, epilogue=None, ahead=None) -> SparseConvTensor:
        """``epilogue`` = (scale [oC] fp32 or None, shift [oC] fp32 or None, relu): applied to the
        accumulators before the store, inference only (no autograd through it; no reference
        counterpart).  ``ahead``: the result of :meth:`count_ahead` on a tensor with this input's
        coordinates (no reference counterpart either)."""
        assert self.in_channels == input.C, \
            "input channel does not match Expect: {}, got {}".format(self.in_channels, input.C)
        in_shape = [input.D, input.W, input.H]
        out_shape = in_shape if self.subm else out_spatial(in_shape, self.kernel_size, self.stride,
                                                            self.padding, self.dilation)
        weight = self.weight.view(-1, self.in_channels, self.out_channels)
        training = torch.is_grad_enabled() and (weight.requires_grad or input.feature.requires_grad)
        oz_idx, oz_ptr, book, rule_size, tile_grid_shape = self._rules(
            input, out_shape, ahead, keep=training or self.indice_key is not None, training=training)
        self.rule_book = book if isinstance(book, RuleBook) else None
        if epilogue is not None:
            if training:
                raise RuntimeError("a fused epilogue has no backward: call under torch.no_grad()")
            scale, shift, relu = epilogue
            w = weight if weight.dtype == input.feature.dtype else weight.to(input.feature.dtype)
            out_feature = ext.rule_conv(input.feature, w, book, rule_size, oz_idx.shape[0], scale, shift,
                                        bool(relu), cache_packed=not self.training and w is weight)
        elif not training:
            w = weight if weight.dtype == input.feature.dtype else weight.to(input.feature.dtype)
            out_feature = ext.rule_conv(input.feature, w.detach(), book, rule_size, oz_idx.shape[0],
                                        cache_packed=not self.training and w is weight)
        else:
            out_feature = ConvFunction.apply(input.feature, weight, book, rule_size, tile_grid_shape,
                                             oz_idx.shape[0])
        out = SparseConvTensor(out_feature, out_shape, input.B, z_ptr=oz_ptr, z_idx=oz_idx)
        out.rule_cache = input.rule_cache
        # the rows' columns, where known: the input's own for a submanifold layer, a by-product of the
        # output-coordinate kernels for a strided one
        out.row_cols = book.out_row_cols if isinstance(book, RuleBook) else None
        return out


SparseConv3d = Conv3d


class SubMConv3d(Conv3d):
    """Submanifold convolution: outputs live exactly at the input sites; padding is
    forced to K//2 whatever is passed (conv.py:200-210)."""

    def __init__(self, in_channels, out_channels, kernel_size=3, stride=1, padding=0, dilation=1,
                 groups=1, bias=False, subm=False, indice_key=None, **kwargs):
        super().__init__(in_channels, out_channels, kernel_size, subm=True, stride=stride,
                         padding=padding, dilation=dilation, groups=groups, bias=bias,
                         indice_key=indice_key, **kwargs)
        self.padding = tuple(k // 2 for k in self.kernel_size)
