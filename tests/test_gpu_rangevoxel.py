"""GPU parity of xyz2RangeVoxel (sph_xyz_to_rangevoxel through sphconv_amd.data) against the
numpy restatement of the reference (oracle.xyz2rangevoxel, reference sphconv/data.py:75-128).

The bins come out of float32 sqrt / acos / asin / log; the device's and numpy's versions of
those functions may differ in the last bit, which can move a point that sits within a few
float32 ulps of a bin boundary.  So: bins must be equal except where the oracle's unclamped
float bin is within 1e-3 of an integer (and at most 0.1 % of the points may differ at all);
everything after the bins is integer work and must be bit-exact given the bins."""
import os

import numpy as np
import pytest
import torch

import sphconv_amd as sphconv
from oracle import oracle as O
from sphconv_amd.data import range_params

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
KITTI = os.path.join(HERE, "golden", "kitti_000000_reduced.bin")   # reference test/000000.bin


def _check(pts, **kw):
    rv, idx = sphconv.xyz2RangeVoxel(pts, return_indices=True, **kw)
    f, d, t, bins, raw = O.xyz2rangevoxel(pts, **kw)
    got = idx.cpu().numpy()
    with np.errstate(invalid="ignore"):
        near = np.abs(raw - np.rint(raw)) < 1e-3
    near |= ~np.isfinite(raw)
    differ = got != bins
    assert (~differ | near).all()
    assert differ.any(axis=1).mean() <= 1e-3
    # integer part: scatter of the device's own bins, later point wins
    v_res, h_res = rv.thick.shape[1], rv.thick.shape[2]
    ef = np.zeros((1, pts.shape[1], 1, v_res, h_res), np.float32)
    ed = np.zeros((1, 1, v_res, h_res), np.int32)
    et = np.zeros((1, v_res, h_res), np.int32)
    for i in range(pts.shape[0]):
        ef[0, :, 0, got[i, 0], got[i, 1]] = pts[i]
        ed[0, 0, got[i, 0], got[i, 1]] = got[i, 2]
        et[0, got[i, 0], got[i, 1]] = 1
    assert np.array_equal(rv.feature.cpu().numpy(), ef)
    assert np.array_equal(rv.depth.cpu().numpy(), ed) and np.array_equal(rv.thick.cpu().numpy(), et)
    if not differ.any():
        assert np.array_equal(ef, f) and np.array_equal(ed, d) and np.array_equal(et, t)
    return rv


def test_kitti_scan_default_and_linear_depth():
    pts = np.fromfile(KITTI, dtype=np.float32).reshape(-1, 4)
    rv = _check(pts)
    assert tuple(rv.shape) == (1, 4, 512, 64, 512)
    _check(pts, log=False)
    _check(pts, v_res=32, h_res=1024, d_res=64, v_range=(85.0, 110.0), h_range=(-60, 60), d_range=(2, 80.0))


def test_degenerate_points_and_empty_cloud():
    th, ph = np.radians(95.0), np.radians(1.0)
    same = [[(10 + i) * np.sin(th) * np.cos(ph), (10 + i) * np.sin(th) * np.sin(ph), (10 + i) * np.cos(th), i]
            for i in range(5)]
    pts = np.array(same + [[0, 0, 5, 1], [0, 0, 0, 2], [1e-3, 0, 0, 3], [500, 400, -300, 4], [-20, 1, 0.5, 5]],
                   np.float32)
    _check(pts)
    rv = sphconv.xyz2RangeVoxel(np.zeros((0, 4), np.float32))
    assert int(rv.thick.sum()) == 0 and float(rv.feature.abs().sum()) == 0.0


def test_batch_merge_feeds_the_convolution():
    pts = np.fromfile(KITTI, dtype=np.float32).reshape(-1, 4)
    gen = sphconv.VoxelGenerator(64, 512, 64, (87.5, 103.4), (-45, 45), (6, 70.4), True)
    a, b = gen.generate(pts), gen.generate(pts[::2] * np.float32(1.01))
    batch = sphconv.merge_rangevoxel_batch([a, b])
    assert tuple(batch.shape) == (2, 4, 64, 64, 512) and batch.feature.shape[0] == 2
    x = batch.to_sparse()
    n = int(batch.thick.sum())
    assert x.feature.shape == (n, 4)
    conv = sphconv.SubMConv3d(4, 16, 3).cuda()
    y = conv(x)
    assert y.feature.shape == (n, 16) and torch.isfinite(y.feature).all()
    dense = batch.dense()
    assert tuple(dense.shape) == (2, 4, 64, 64, 512)
    assert int((dense.abs().sum(1) > 0).sum()) <= n
