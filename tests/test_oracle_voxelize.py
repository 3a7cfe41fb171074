"""Pins of the restatement of the reference's voxeliser (oracle.system_transform, voxel_cells,
voxelize_cells, points_to_voxel_v2, simple_voxel; reference include/point2voxel.h:412-512,
sphconv/utils/coord_transform.py, sphconv/utils/voxelize.py:126-214, sphconv/vfe.py:210-228):
hand-worked voxel lists for the sequential rules, closed-form coordinates, and invariants on the
reduced KITTI scan the reference's tests hold."""
import os

import numpy as np
import pytest

from oracle import oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
KITTI = os.path.join(HERE, "golden", "kitti_000000_reduced.bin")   # reference test/000000.bin
RANGE, SRANGE = [6, -40, -3, 70.4, 40, 1], [6, -45, 87.5, 70.4, 45, 100]


def test_sequential_rules_by_hand():
    # cells of 8 points: A B A C (outside) B A D ; max_points 2, max_voxels 3
    cells = np.array([[0, 0, 1], [0, 0, 2], [0, 0, 1], [0, 1, 0], [9, 9, 9], [0, 0, 2], [0, 0, 1], [1, 1, 1]])
    valid = np.array([1, 1, 1, 1, 0, 1, 1, 1], bool)
    pts = np.arange(32, dtype=np.float32).reshape(8, 4)
    sp = pts + 100
    res = O.voxelize_cells(pts, sp, cells, valid, max_points=2, max_voxels=3)
    # voxels in order of first appearance: A, B, C; D would be the 4th: the loop stops at point 7
    assert res["voxel_num"] == 3
    assert res["coordinates"][:3].tolist() == [[0, 0, 1], [0, 0, 2], [0, 1, 0]]
    assert res["num_points_per_voxel"][:3].tolist() == [2, 2, 1]          # A's third point (6) is dropped
    assert np.array_equal(res["voxels"][0], pts[[0, 2]]) and np.array_equal(res["voxels"][1], pts[[1, 5]])
    assert np.array_equal(res["voxels"][2, 0], pts[3]) and (res["voxels"][2, 1] == 0).all()
    assert res["voxel_point_mask"][:3, :, 0].tolist() == [[1, 1], [1, 1], [1, 0]]
    # the stop drops later points even of open voxels: with max_voxels 2 the loop ends at point 3 (C)
    res = O.voxelize_cells(pts, sp, cells, valid, max_points=3, max_voxels=2)
    assert res["voxel_num"] == 2 and res["num_points_per_voxel"][:2].tolist() == [2, 1]
    # append modes
    res = O.voxelize_cells(pts, sp, cells, valid, 1, 8, append_mode=1)
    assert res["voxels"].shape[2] == 7 and np.array_equal(res["voxels"][0, 0], np.r_[pts[0], sp[0, :3]])
    res = O.voxelize_cells(pts, sp, cells, valid, 1, 8, append_mode=2)
    assert np.array_equal(res["voxels"][1, 0], np.r_[sp[1, :3], pts[1, 3]])


@pytest.mark.parametrize("system", ["spherical", "l-spherical", "cylinder", "l-cylinder", "hybrid", "l-hybrid"])
def test_coordinates_closed_form(system):
    r, theta, phi = 20.0, np.radians(95.0), np.radians(10.0)
    p = np.array([[r * np.sin(theta) * np.cos(phi), r * np.sin(theta) * np.sin(phi), r * np.cos(theta), 0.25]], np.float32)
    sp, rng = O.system_transform(p, RANGE, SRANGE, system)
    d = r * np.sin(theta)
    want0 = {"spherical": r, "l-spherical": np.log(r), "cylinder": d, "l-cylinder": np.log(d), "hybrid": d,
             "l-hybrid": np.log(d)}[system]
    want2 = r * np.cos(theta) if "cylinder" in system else theta
    np.testing.assert_allclose(sp[0], [want0, phi, want2, 0.25], rtol=1e-5)
    lo0 = np.log(6) if system.startswith("l-") else 6
    hi0 = np.log(70.4) if system.startswith("l-") else 70.4
    lo2, hi2 = (-3, 1) if "cylinder" in system else (np.radians(87.5), np.radians(100))
    np.testing.assert_allclose(rng, [lo0, np.radians(-45), lo2, hi0, np.radians(45), hi2], rtol=1e-12)
    # bins of this point on a [64, 90, 25] grid
    coor, ok, _ = O.voxel_cells(sp, rng, [64, 90, 25])
    b0 = int((want0 - lo0) / ((hi0 - lo0) / 64)); b1 = int((10 + 45) / 1.0); b2 = int((want2 - lo2) / ((hi2 - lo2) / 25))
    assert ok[0] and coor[0].tolist() == [b2, b1, b0]


def test_kitti_scan_invariants_and_mean():
    pts = np.fromfile(KITTI, dtype=np.float32).reshape(-1, 4)
    res = O.points_to_voxel_v2(pts, RANGE, SRANGE, 2, 24000, [512, 512, 64], "spherical")
    m = res["voxel_num"]
    sp, rng = O.system_transform(pts, RANGE, SRANGE, "spherical")
    coor, ok, _ = O.voxel_cells(sp, rng, [512, 512, 64])
    key = (coor[:, 0] * 512 + coor[:, 1]) * 512 + coor[:, 2]
    uniq, first, counts = np.unique(key[ok], return_index=True, return_counts=True)
    assert m == uniq.shape[0] < 24000
    order = np.argsort(first)                                   # voxels in order of first appearance
    got_key = (res["coordinates"][:m, 0].astype(np.int64) * 512 + res["coordinates"][:m, 1]) * 512 + res["coordinates"][:m, 2]
    assert np.array_equal(got_key, uniq[order])
    assert np.array_equal(res["num_points_per_voxel"][:m], np.minimum(counts[order], 2))
    assert (res["coordinates"][:m].max(0) < [64, 512, 512]).all() and (res["coordinates"][:m] >= 0).all()
    idx_valid = np.nonzero(ok)[0]
    assert np.array_equal(res["voxels"][:m, 0], pts[idx_valid[first[order]]])     # first point of every voxel
    assert (res["voxels"][m:] == 0).all() and (res["num_points_per_voxel"][m:] == 0).all()
    mean = O.simple_voxel(res["voxels"][:m], res["num_points_per_voxel"][:m])
    one = res["num_points_per_voxel"][:m] == 1
    assert np.array_equal(mean[one], res["voxels"][:m][one, 0])
    np.testing.assert_allclose(mean[~one], res["voxels"][:m][~one].mean(1), rtol=1e-6)


def test_sphere_branch_without_resolution_closed_form():
    """oracle.points_to_voxel_sphere (point2voxel.h:316-399): grid = round(range / voxel size); a point at
    the centre of bin (it, ip, ir) of (theta, phi, log r) gets exactly these coordinates, in that order;
    points outside any of the three ranges are skipped; the rest is the shared sequential loop."""
    vs = [0.25, 0.5, 2.0]                         # log r, degrees, degrees
    srange = [1.0, -45.0, 80.0, 4.0, 45.0, 100.0]  # log r from 1 to 4, phi, theta
    want_grid = [12, 180, 10]
    bins = [(0, 0, 0), (9, 179, 11), (3, 90, 5), (3, 90, 5), (7, 12, 2)]
    pts = []
    for it, ip, ir in bins:
        theta = np.radians(80.0 + (it + 0.5) * 2.0)
        phi = np.radians(-45.0 + (ip + 0.5) * 0.5)
        r = np.exp(1.0 + (ir + 0.5) * 0.25)
        pts.append([r * np.sin(theta) * np.cos(phi), r * np.sin(theta) * np.sin(phi), r * np.cos(theta), len(pts)])
    outside = [[np.exp(0.5), 0.0, 0.0, 9.0],                       # log r below the range
               [-10.0, 0.1, 0.0, 9.0],                             # x < 0: asin folds phi back, theta = 90 is inside -> kept
               [10.0 * np.cos(np.radians(60)), 10.0 * np.sin(np.radians(60)), 0.0, 9.0],   # phi = 60 degrees
               [10.0 * np.sin(np.radians(70)), 0.0, 10.0 * np.cos(np.radians(70)), 9.0]]   # theta = 70 degrees
    allp = np.array(pts + outside, np.float32)
    res = O.points_to_voxel_sphere(allp, vs, srange, max_points=2, max_voxels=10)
    assert res["grid_size"] == want_grid
    # four distinct cells among the five centred points (the third and fourth share one), plus the folded point
    assert res["voxel_num"] == 5
    assert res["coordinates"][:4].tolist() == [list(bins[0]), list(bins[1]), list(bins[2]), list(bins[4])]
    assert res["num_points_per_voxel"][:5].tolist() == [1, 1, 2, 1, 1]
    assert np.array_equal(res["voxels"][2], allp[[2, 3]])
    # the folded point: phi = asin(0.1 / 10.0005) ~ 0.573 degrees -> bin 91, theta 90 -> bin 5, log 10 = 2.3026 -> bin 5
    assert res["coordinates"][4].tolist() == [5, 91, 5]
    # rounding of the grid: 2.2 / 0.5 = 4.4 -> 4, 2.3 / 0.5 = 4.6 -> 5, exact halves go away from zero (C round)
    g = O.points_to_voxel_sphere(allp[:1], [0.5, 0.5, 0.5], [0, 0, 0, 2.2, 2.3, 1.25], 1, 1)["grid_size"]
    assert g == [4, 5, 3]
