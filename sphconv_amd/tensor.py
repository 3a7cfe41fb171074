"""Sparse tensor in the reference's per-column compressed layout
(sphconv/tensor.py:33-125)."""
from typing import List, Optional

import torch

from .functional import InitTensorFunction, ToDenseFunction


class SparseTensorBase:
    def __init__(self, B, D, W, H, C, device, dtype, itype, feature, z_idx, z_ptr):
        self.B, self.D, self.W, self.H, self.C = B, D, W, H, C
        self.device, self.dtype, self.itype = device, dtype, itype
        self.feature, self.z_idx, self.z_ptr = feature, z_idx, z_ptr


class SparseConvTensor(SparseTensorBase):
    """``feature [NNZ,C]`` rows, ``z_idx [NNZ]`` their coordinate on the compressed
    axis, ``z_ptr [B,S0,S1]`` inclusive prefix sums of per-column row counts.
    ``spatial_shape_DWH = [S0,S1,S2]`` (the reference calls them D, W, H); COO
    ``indices`` rows are (b, s0, s1, s2).  Either pass ``indices`` (rows get
    reordered) or ready ``z_idx``/``z_ptr``."""

    def __init__(self, raw_feature: torch.Tensor, spatial_shape_DWH: List[int], batch_size: int,
                 indices: Optional[torch.Tensor] = None, z_idx: Optional[torch.Tensor] = None,
                 z_ptr: Optional[torch.Tensor] = None, row_cols: Optional[torch.Tensor] = None):
        self.rule_cache = {}
        # optional int32 [NNZ]: the column (index into the flattened z_ptr) of every row.  The reference's kernels
        # get it from their launch geometry (one thread per column, rules.cu:256-259); here the rule kernel
        # searches z_ptr for it unless the tensor brings it along.  Tensors made from COO indices and the outputs
        # of convolutions carry it; ``with_row_cols()`` adds it to a tensor made from bare z_idx / z_ptr.
        self.row_cols = row_cols
        self.requires_grad = False
        s0, s1, s2 = (int(v) for v in spatial_shape_DWH)
        if z_idx is not None and z_ptr is not None:
            super().__init__(batch_size, s0, s1, s2, raw_feature.shape[-1], raw_feature.device,
                             raw_feature.dtype, z_idx.dtype, raw_feature, z_idx, z_ptr)
            return
        if indices is None:
            raise ValueError("SparseConvTensor needs either indices or z_idx and z_ptr")
        assert indices.dtype == torch.int32
        assert indices.dim() == 2 and indices.shape[1] == 4
        assert raw_feature.dim() == 2 and raw_feature.shape[0] == indices.shape[0]
        assert raw_feature.device == indices.device
        super().__init__(batch_size, s0, s1, s2, raw_feature.shape[-1], raw_feature.device,
                         raw_feature.dtype, indices.dtype, None, None, None)
        self.feature, self.z_idx, self.z_ptr = InitTensorFunction.apply(
            raw_feature, indices, self.B, [self.D, self.W, self.H])
        if self.z_ptr.is_cuda:
            self.with_row_cols()

    def with_row_cols(self):
        """Computes ``row_cols`` from ``z_ptr`` (one small kernel) if the tensor does not have it yet."""
        if self.row_cols is None and self.z_ptr is not None and self.z_ptr.is_cuda:
            from .rulebook import row_columns
            self.row_cols = row_columns(self.z_ptr, int(self.z_idx.shape[0]))
        return self

    @property
    def shape(self):
        # tensor.py:104-106 reports [B,C,D,H,W]; kept for compatibility
        return [self.B, self.C, self.D, self.H, self.W]

    @property
    def spatial_shape(self):
        return [self.D, self.W, self.H]

    def find_rule(self, key: str):
        if key is None:
            return None
        return self.rule_cache.get(key)

    def dense(self, device=None):
        """Dense [B,C,S0,S1,S2] copy, zeros at inactive cells."""
        out = ToDenseFunction.apply(self.feature, self.z_idx, self.z_ptr,
                                    [self.B, self.C, self.D, self.W, self.H])
        return out if device is None else out.to(device)
