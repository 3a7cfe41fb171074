"""Pins of the numpy restatement of xyz2RangeVoxel (oracle.xyz2rangevoxel, reference
sphconv/data.py:75-128): closed-form bins of points placed at chosen spherical coordinates,
clamping, the later-point-wins rule, and the reduced KITTI scan the reference's tests hold."""
import os

import numpy as np
import pytest

from oracle import oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
KITTI = os.path.join(HERE, "golden", "kitti_000000_reduced.bin")   # reference test/000000.bin


def _point(r, theta_deg, phi_deg, extra=0.5):
    th, ph = np.radians(theta_deg), np.radians(phi_deg)
    return [r * np.sin(th) * np.cos(ph), r * np.sin(th) * np.sin(ph), r * np.cos(th), extra]


def test_bins_of_points_at_chosen_angles():
    # bin centres are far from any boundary, so float32 rounding cannot move them
    v_res, h_res, d_res = 64, 512, 512
    v_range, h_range, d_range = (87.5, 103.4), (-45, 45), (6, 70.4)
    want, pts = [], []
    for ti, pi, di in [(0, 0, 0), (10, 256, 106), (63, 511, 511), (31, 100, 300), (5, 400, 17)]:
        theta = v_range[0] + (ti + 0.5) * (v_range[1] - v_range[0]) / v_res
        phi = h_range[0] + (pi + 0.5) * (h_range[1] - h_range[0]) / h_res
        r = np.exp(np.log(d_range[0]) + (di + 0.5) * (np.log(d_range[1]) - np.log(d_range[0])) / d_res)
        pts.append(_point(r, theta, phi))
        want.append((ti, pi, di))
    bins = O.xyz2rangevoxel(np.array(pts, np.float32), v_res, h_res, d_res, v_range, h_range, d_range, True)[3]
    assert bins.tolist() == [list(w) for w in want]
    # linear depth
    pts = [_point(6 + (di + 0.5) * (70.4 - 6) / 512, 95.0, 3.0) for di in (0, 77, 511)]
    bins = O.xyz2rangevoxel(np.array(pts, np.float32), log=False)[3]
    assert bins[:, 2].tolist() == [0, 77, 511]


def test_clamping_and_degenerate_points():
    pts = np.array([_point(1.0, 95, 0),        # nearer than the range: depth bin 0
                    _point(500.0, 95, 0),      # farther: last bin
                    _point(20.0, 60, 0),       # above the polar range: row 0
                    _point(20.0, 140, 0),      # below: last row
                    _point(20.0, 95, -80),     # azimuth outside: column 0
                    _point(20.0, 95, 80),      # last column
                    [0.0, 0.0, 5.0, 1.0]],     # on the z axis: asin(0/0) is NaN -> column 0
                   np.float32)
    bins = O.xyz2rangevoxel(pts)[3]
    assert bins[0, 2] == 0 and bins[1, 2] == 511
    assert bins[2, 0] == 0 and bins[3, 0] == 63
    assert bins[4, 1] == 0 and bins[5, 1] == 511
    assert bins[6, 1] == 0 and bins[6, 0] == 0


def test_later_point_wins_and_scatter_invariants():
    rng = np.random.default_rng(0)
    pts = np.array([_point(10 + i, 95.0, 1.0, extra=i) for i in range(5)], np.float32)   # same pixel
    f, d, t, bins, _ = O.xyz2rangevoxel(pts)
    assert len({(b[0], b[1]) for b in bins.tolist()}) == 1
    ti, pi = bins[0, 0], bins[0, 1]
    assert f[0, 3, 0, ti, pi] == 4.0 and d[0, 0, ti, pi] == bins[4, 2] and t.sum() == 1
    pts = np.fromfile(KITTI, dtype=np.float32).reshape(-1, 4)
    f, d, t, bins, _ = O.xyz2rangevoxel(pts)
    pix = bins[:, 0].astype(np.int64) * 512 + bins[:, 1]
    assert t.sum() == np.unique(pix).shape[0]
    last = {}
    for i, p in enumerate(pix.tolist()):
        last[p] = i
    for p, i in list(last.items())[::97]:
        assert np.array_equal(f[0, :, 0, p // 512, p % 512], pts[i]) and d[0, 0, p // 512, p % 512] == bins[i, 2]
    assert (f[0, :, 0][:, t[0] == 0] == 0).all() and (d[0, 0][t[0] == 0] == 0).all()


def test_kitti_scan_against_float64():
    """float32 bins equal the float64 evaluation of the same formulas except within a few
    float32 ulps of a bin boundary."""
    pts = np.fromfile(KITTI, dtype=np.float32).reshape(-1, 4)
    bins, raw = O.xyz2rangevoxel(pts)[3:]
    p = pts.astype(np.float64)
    r = np.sqrt((p[:, :3] ** 2).sum(1))
    tf = (np.arccos(p[:, 2] / r) - np.radians(87.5)) / (np.radians(15.9) / 64)
    pf = (np.arcsin(p[:, 1] / np.hypot(p[:, 0], p[:, 1])) - np.radians(-45)) / (np.radians(90) / 512)
    df = (np.log(r) - np.log(6)) / ((np.log(70.4) - np.log(6)) / 512)
    ref = np.stack([np.clip(np.trunc(tf), 0, 63), np.clip(np.trunc(pf), 0, 511), np.clip(np.trunc(df), 0, 511)], 1)
    near = np.abs(np.stack([tf, pf, df], 1) - np.rint(np.stack([tf, pf, df], 1))) < 2e-3
    assert ((bins == ref) | near).all()
    assert (bins != ref).mean() < 2e-3
