"""Point cloud -> RangeVoxel (reference: sphconv/data.py).

``xyz2RangeVoxel`` keeps the reference's signature and defaults (data.py:28-38); the
conversion itself runs on the GPU in float32, operation by operation as the reference's
numpy code does on float32 points (data.py:75-104), and points that share a pixel are
resolved the way its indexed assignment does: the later point wins (data.py:106-121).
"""
import ctypes as C
import math
from typing import List

import numpy as np
import torch

from . import _lib as L
from .rangevoxel import RangeVoxel


def _f32(x) -> float:
    return float(np.float32(x))


def range_params(v_res, h_res, d_res, v_range, h_range, d_range, log):
    """The float32 constants of data.py:85-97 (numpy scalars enter float32 arithmetic rounded
    to float32): (v0, h0, dtheta, dphi, d0, dr)."""
    dphi = np.radians(h_range[1] - h_range[0]) / h_res
    dtheta = np.radians(v_range[1] - v_range[0]) / v_res
    if log:
        d0 = np.log(d_range[0])
        dr = (np.log(d_range[1]) - np.log(d_range[0])) / d_res
    else:
        d0 = d_range[0]
        dr = (d_range[1] - d_range[0]) / d_res
    return (_f32(np.radians(v_range[0])), _f32(np.radians(h_range[0])), _f32(dtheta), _f32(dphi), _f32(d0), _f32(dr))


def xyz2RangeVoxel(points,
                   v_res=64,
                   h_res=512,
                   d_res=512,
                   v_range=(87.5, 103.4),
                   h_range=(-45, 45),
                   d_range=(6, 70.4),
                   log=True,
                   verbose=False,
                   device=None,
                   return_indices=False) -> RangeVoxel:
    """data.py:28-128.  ``points`` [M,NDim] (numpy or torch, x, y, z first) of one frame ->
    RangeVoxel with feature [1,NDim,1,v_res,h_res], depth [1,1,v_res,h_res], thick
    [1,v_res,h_res], shape (1,NDim,d_res,v_res,h_res), on ``device`` (default: the points'
    device if they are a GPU tensor, else the current GPU).  ``return_indices`` also returns
    each point's (theta, phi, depth) bins [M,3]."""
    if isinstance(points, np.ndarray):
        points = torch.from_numpy(np.ascontiguousarray(points, dtype=np.float32))
    if points.dim() != 2 or points.shape[1] < 3:
        raise ValueError("points must be [M,NDim] with x, y, z first")
    if device is None:
        device = points.device if points.is_cuda else torch.device("cuda", torch.cuda.current_device())
    pts = points.to(device=device, dtype=torch.float32).contiguous()
    m, ndim = pts.shape
    v0, h0, dtheta, dphi, d0, dr = range_params(v_res, h_res, d_res, v_range, h_range, d_range, log)
    feature = torch.empty((1, ndim, 1, v_res, h_res), dtype=torch.float32, device=device)
    depth = torch.empty((1, 1, v_res, h_res), dtype=torch.int32, device=device)
    thick = torch.empty((1, v_res, h_res), dtype=torch.int32, device=device)
    winner = torch.empty(v_res * h_res, dtype=torch.int32, device=device)
    idx = torch.empty((m, 3), dtype=torch.int32, device=device) if return_indices else None
    with torch.cuda.device(device):
        L.check(L.lib().sph_xyz_to_rangevoxel(L.ptr(pts) if m else None, m, ndim, int(v_res), int(h_res), int(d_res),
                                              v0, h0, dtheta, dphi, d0, dr, int(bool(log)), L.ptr(winner),
                                              L.ptr(feature), L.ptr(depth), L.ptr(thick), L.ptr(idx), L.stream()))
    rv = RangeVoxel(feature, depth, thick, shape=(1, ndim, d_res, v_res, h_res))
    return (rv, idx) if return_indices else rv


class VoxelGenerator(object):
    """A fixed range-image geometry, applied to point clouds with ``generate`` (same constructor arguments and
    attributes as data.py:12-26: resolutions, then ranges, then the log-depth switch)."""

    _FIELDS = ("v_res", "h_res", "d_res", "v_range", "h_range", "d_range", "log")

    def __init__(self, v_res, h_res, d_res, v_range, h_range, d_range, log):
        for name, value in zip(self._FIELDS, (v_res, h_res, d_res, v_range, h_range, d_range, log)):
            setattr(self, name, value)

    def generate(self, points):
        return xyz2RangeVoxel(points, *(getattr(self, name) for name in self._FIELDS))


def merge_rangevoxel_batch(voxel_list: List[RangeVoxel]) -> RangeVoxel:
    """data.py:133-150: concatenates frames of the same shape along the batch axis."""
    feature = torch.cat([x.feature for x in voxel_list], dim=0)
    depth = torch.cat([x.depth for x in voxel_list], dim=0)
    thick = torch.cat([x.thick for x in voxel_list], dim=0)
    shape = list(voxel_list[0].shape)
    shape[0] = len(voxel_list)
    return RangeVoxel(feature, depth, thick, shape=shape)
