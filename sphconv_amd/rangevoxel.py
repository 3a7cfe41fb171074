"""Legacy range-voxel container (reference: sphconv/rangevoxel.py:5-95) with a
working bridge to the compressed layout the convolutions use.

feature [B,C,T,H,W], depth [B,T,H,W] (int, S2 coordinate of slot t), thick
[B,H,W] (int, number of used slots per column), shape (B,C,D,H,W).  Slot t of
column (b,h,w) is active iff t < thick[b,h,w].
"""
import torch

from .tensor import SparseConvTensor


def check_size(shape, feature_shape, depth_shape, thick_shape):
    """rangevoxel.py:71-95"""
    B, C, D, H, W = shape
    B_f, C_f, T_f, H_f, W_f = feature_shape
    B_d, T_d, H_d, W_d = depth_shape
    B_t, H_t, W_t = thick_shape
    msg = "feature.shape={}, depth.shape={}, thick.shape={},  shape={}".format(
        feature_shape, depth_shape, thick_shape, shape)
    assert B == B_d == B_t == B_f, "batch dimension not match, " + msg
    assert H == H_d == H_t == H_f, "hight dimension not match, " + msg
    assert W == W_d == W_t == W_f, "width dimension not match, " + msg
    assert C == C_f, "channel dimension not match, " + msg
    assert T_d == T_f, "thick dimension not match, " + msg


class RangeVoxel(object):
    def __init__(self, feature: torch.Tensor, depth, thick, shape):
        check_size(shape, feature.shape, depth.shape, thick.shape)
        self.feature = feature
        self.depth = depth
        self.thick = thick
        self.shape = shape
        self.indice_dict = {}

    def cuda(self):
        self.feature = self.feature.cuda()
        self.depth = self.depth.cuda()
        self.thick = self.thick.cuda()
        return self

    def find_indice_pair(self, key):
        if key is None:
            return None
        return self.indice_dict.get(key)

    def to_sparse(self) -> SparseConvTensor:
        """Compressed form with S0=H, S1=W, S2=D (the depth axis is the compressed one)."""
        B, C, D, H, W = self.shape
        T = self.depth.shape[1]
        active = torch.arange(T, device=self.thick.device)[None, :, None, None] < self.thick[:, None].long()
        b, t, h, w = active.nonzero(as_tuple=True)
        indices = torch.stack([b, h, w, self.depth[b, t, h, w].long()], dim=1).to(torch.int32)
        rows = self.feature[b, :, t, h, w]
        return SparseConvTensor(rows.contiguous(), [H, W, D], B, indices=indices.contiguous())

    def dense(self, device=None):
        """Dense [B,C,D,H,W] tensor (the reference's own ``dense`` calls ToDenseFunction
        with a stale signature, rangevoxel.py:61-69; this one goes through the
        compressed form)."""
        out = self.to_sparse().dense().permute(0, 1, 4, 2, 3).contiguous()  # [B,C,H,W,D] -> [B,C,D,H,W]
        return out if device is None else out.to(device)

    @staticmethod
    def from_sparse(x: SparseConvTensor) -> "RangeVoxel":
        B, H, W, D = x.B, x.D, x.W, x.H
        counts = torch.diff(x.z_ptr.reshape(-1).long(), prepend=x.z_ptr.new_zeros(1).long())
        T = max(int(counts.max().item()) if counts.numel() else 0, 1)
        col = torch.repeat_interleave(torch.arange(counts.numel(), device=counts.device), counts)
        start = (x.z_ptr.reshape(-1).long() - counts)[col]
        slot = torch.arange(col.numel(), device=col.device) - start
        b = torch.div(col, H * W, rounding_mode="floor")
        h = torch.div(col % (H * W), W, rounding_mode="floor")
        w = col % W
        feature = x.feature.new_zeros((B, x.C, T, H, W))
        depth = torch.zeros((B, T, H, W), dtype=torch.int32, device=col.device)
        feature[b, :, slot, h, w] = x.feature
        depth[b, slot, h, w] = x.z_idx
        return RangeVoxel(feature, depth, counts.view(B, H, W).to(torch.int32), (B, x.C, D, H, W))
