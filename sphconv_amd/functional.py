"""Autograd functions of the sparse convolution path, with the reference's
names and signatures (sphconv/functional.py:12-131)."""
from typing import List

import torch

from . import sphconv_cuda as ext
from .rulebook import RuleBook


class ConvFunction(torch.autograd.Function):
    """out = rule_conv(feature, weight[KV,iC,oC], rules) with dgrad / wgrad
    (functional.py:48-78).  ``rules`` is a RuleBook (fast path) or the reference's
    padded tensor together with ``rule_size``."""

    @staticmethod
    def forward(ctx, feature, weight, rules, rule_size, tile_grid_shape: List[int], outNNZ: int, packed=None):
        if (ctx.needs_input_grad[0] or ctx.needs_input_grad[1]) and weight.shape[1] > ext.MAX_TRAIN_CHANNELS:
            # forward alone takes up to 256 input channels; say so here, not from inside backward()
            raise ext.L.SphconvError("training takes 1..%d input channels (forward alone up to %d), got %d"
                                     % (ext.MAX_TRAIN_CHANNELS, ext.MAX_FORWARD_IN_CHANNELS, weight.shape[1]))
        book = rules if isinstance(rules, RuleBook) else RuleBook.from_padded(
            rules, rule_size, feature.shape[0], int(outNNZ))
        ctx.save_for_backward(feature, weight)
        ctx.book = book
        ctx.tile_grid_shape = tile_grid_shape
        if packed is not None and weight.dtype != feature.dtype:
            packed = None                       # packed in the weight's type, the kernel needs the feature's
        book.keep = True                        # backward walks the book
        return ext.rule_conv(feature, weight, book, None, outNNZ, packed=packed)

    @staticmethod
    def backward(ctx, d_featureOut):
        feature, weight = ctx.saved_tensors
        book = ctx.book
        d_out = d_featureOut.contiguous()
        if d_out.dtype != feature.dtype:
            d_out = d_out.to(feature.dtype)
        d_feature = d_weight = None
        if ctx.needs_input_grad[0]:
            w = weight if weight.dtype == feature.dtype else weight.to(feature.dtype)
            # contraction over oC with W[k]^T: packed straight from [KV,iC,oC], no permuted copy
            buf, reverse = ext._dgrad_buffers(book, d_out, w.shape[2], w.shape[1])
            if buf is None:
                buf = book.transposed()
            packed = ext._packed_weight(w, True, reverse)
            d_feature = ext._apply(d_out, packed, w.shape[2], w.shape[1], buf)
        if ctx.needs_input_grad[1]:
            # an fp32 master weight gets its gradient straight from the fp32 reduction, not through a 16-bit type
            want_f32 = weight.dtype == torch.float32
            d_weight = ext.rule_conv_d_weight(feature, d_out, book, None,
                                              torch.float32 if want_f32 else None).to(weight.dtype)
        return d_feature, d_weight, None, None, None, None, None


class ToDenseFunction(torch.autograd.Function):
    """[NNZ,C] rows -> dense [B,C,S0,S1,S2] (functional.py:81-106)."""

    @staticmethod
    def forward(ctx, feature, z_idx, z_ptr, shape: List[int]):
        ctx.save_for_backward(z_idx, z_ptr)
        B, C, S0, S1, S2 = shape
        res = torch.zeros((B, S0, S1, S2, C), device=feature.device, dtype=feature.dtype)
        ext.to_dense(feature, z_idx, z_ptr, S2, res)
        return res.permute(0, 4, 1, 2, 3).contiguous()

    @staticmethod
    def backward(ctx, d_featureOut):
        z_idx, z_ptr = ctx.saved_tensors
        d_feature = ext.to_dense_backward(d_featureOut.permute(0, 2, 3, 4, 1).contiguous(), z_idx, z_ptr)
        return d_feature, None, None, None


class InitTensorFunction(torch.autograd.Function):
    """COO rows -> per-column compressed rows (functional.py:109-131)."""

    @staticmethod
    def forward(ctx, raw_feature, indices_bzyx, batchsize: int, spatial_shape: List[int]):
        feature_out, z_idx, z_ptr, permutation = ext.init_tensor(raw_feature, indices_bzyx, batchsize,
                                                                  spatial_shape)
        ctx.save_for_backward(permutation)
        ctx.mark_non_differentiable(z_idx, z_ptr)
        return feature_out, z_idx, z_ptr

    @staticmethod
    def backward(ctx, d_featureOut, d_zidx, d_zptr):
        permutation, = ctx.saved_tensors
        return ext.init_tensor_backward(d_featureOut, permutation), None, None, None
