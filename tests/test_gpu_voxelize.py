"""GPU parity of the point cloud -> voxel path (sph_points_to_voxel through sphconv_amd.voxelize /
datagen) against the restatement of the reference (oracle.points_to_voxel_v2 ..., reference
include/point2voxel.h:412-512, sphconv/utils/coord_transform.py, sphconv/vfe.py:210-228).

The cells come out of float32 sqrt / acos / asin / log, whose device and numpy versions may differ
in the last bit: cells must be equal except where the oracle's float bin is within 1e-3 of an
integer (at most 0.1 % of the points may differ).  Given cells, everything else -- numbering in
order of first appearance, the first max_points points, the stop at max_voxels -- is integer work
and must be bit-exact, which is checked by feeding the oracle's cells to the device."""
import os

import numpy as np
import pytest
import torch

import sphconv_amd as sphconv
from oracle import oracle as O
from sphconv_amd.datagen import VoxelizationVFE, merge_batch_torch
from sphconv_amd.voxelize import VoxelGeneratorV3, points_to_voxel_v2

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
KITTI = os.path.join(HERE, "golden", "kitti_000000_reduced.bin")   # reference test/000000.bin
RANGE, SRANGE = [6, -40, -3, 70.4, 40, 1], [6, -45, 87.5, 70.4, 45, 100]


def _compare(res, want):
    m = want["voxel_num"]
    assert res["voxel_num"] == m
    for k in ("voxels", "coordinates", "num_points_per_voxel", "voxel_point_mask"):
        assert np.array_equal(res[k].cpu().numpy(), want[k]), k


@pytest.mark.parametrize("system", ["spherical", "l-spherical", "cylinder", "l-cylinder", "hybrid", "l-hybrid"])
@pytest.mark.parametrize("grid,max_points,max_voxels,append_mode", [([512, 512, 64], 2, 24000, 0),
                                                                    ([64, 96, 16], 3, 700, 1),
                                                                    ([16, 16, 4], 5, 30000, 2)])
def test_kitti_scan(system, grid, max_points, max_voxels, append_mode):
    pts = np.fromfile(KITTI, dtype=np.float32).reshape(-1, 4)
    sp, rng = O.system_transform(pts, RANGE, SRANGE, system)
    coor, ok, fb = O.voxel_cells(sp, rng, grid)
    cells = np.where(ok, (coor[:, 0] * grid[1] + coor[:, 1]) * grid[0] + coor[:, 2], -1)
    # 1. cells computed on the device
    res = points_to_voxel_v2(pts, None, RANGE, SRANGE, None, max_points, max_voxels, resolution_HWD=grid,
                             coord_system=system, append_mode=append_mode, return_cells=True)
    got = res["cells"].cpu().numpy()
    with np.errstate(invalid="ignore"):
        near = (np.abs(fb - np.rint(fb)) < 1e-3).any(1) | ~np.isfinite(fb).all(1)
    differ = got != cells
    assert (~differ | near).all() and differ.mean() <= 1e-3
    # 2. integer part, bit-exact on the oracle's cells
    want = O.voxelize_cells(pts, sp, coor, ok, max_points, max_voxels, append_mode)
    res2 = points_to_voxel_v2(pts, None, RANGE, SRANGE, None, max_points, max_voxels, resolution_HWD=grid,
                              coord_system=system, append_mode=append_mode, cells=torch.tensor(cells))
    if append_mode == 0:
        _compare(res2, want)
    else:
        # appended system coordinates are float32 transcendental results: compare those to 1e-6 relative
        assert res2["voxel_num"] == want["voxel_num"]
        for k in ("coordinates", "num_points_per_voxel", "voxel_point_mask"):
            assert np.array_equal(res2[k].cpu().numpy(), want[k]), k
        np.testing.assert_allclose(res2["voxels"].cpu().numpy(), want["voxels"], rtol=2e-6, atol=1e-6)
    if not differ.any() and append_mode == 0:
        _compare({k: v for k, v in res.items() if k != "cells"}, want)


def test_many_points_scan_over_many_workgroups():
    """Eight jittered copies of the reference's scan (about 150 000 points): the voxel numbering and the
    first-point search scan arrays of more than 64 workgroups' worth of elements.  Integer part on the
    oracle's cells, bit-exact."""
    base = np.fromfile(KITTI, dtype=np.float32).reshape(-1, 4)
    rng = np.random.default_rng(3)
    pts = np.concatenate([base + rng.normal(0, 0.05, base.shape).astype(np.float32) for _ in range(8)])
    assert pts.shape[0] > 64 * 2048
    grid, max_points, max_voxels = [512, 512, 64], 3, 200000
    sp, rg = O.system_transform(pts, RANGE, SRANGE, "spherical")
    coor, ok, _ = O.voxel_cells(sp, rg, grid)
    cells = np.where(ok, (coor[:, 0] * grid[1] + coor[:, 1]) * grid[0] + coor[:, 2], -1)
    want = O.voxelize_cells(pts, sp, coor, ok, max_points, max_voxels, 0)
    res = points_to_voxel_v2(pts, None, RANGE, SRANGE, None, max_points, max_voxels, resolution_HWD=grid,
                             coord_system="spherical", append_mode=0, cells=torch.tensor(cells))
    _compare(res, want)
    assert want["voxel_num"] > 30000


@pytest.mark.parametrize("max_points,max_voxels", [(5, 4000), (40, 4000), (3, 300), (1, 1)])
def test_crowded_cells_long_segments_and_the_stop(max_points, max_voxels):
    """Synthetic cells: a third of 20 000 points share one cell and a tenth another (segments of thousands of
    points, which a wave walks together), the rest spread over 3000 cells with hash collisions among them, one
    point in 50 outside the grid; with 300 voxels (and with one) the reference's loop stops in the middle of the list.
    Bit-exact against the sequential loop on the same cells."""
    rng = np.random.default_rng(max_points * 1000 + max_voxels)
    n, grid = 20000, [64, 64, 8]
    ncell = grid[0] * grid[1] * grid[2]
    pool = rng.choice(ncell, 3000, replace=False)
    cells = pool[rng.integers(0, 3000, n)]
    u = rng.random(n)
    cells = np.where(u < 0.33, pool[0], np.where(u < 0.43, pool[1], cells))
    cells = np.where(rng.random(n) < 0.02, -1, cells).astype(np.int64)
    pts = rng.normal(0, 10, (n, 4)).astype(np.float32)
    ok = cells >= 0
    c = np.where(ok, cells, 0)
    coor = np.stack([c // (grid[0] * grid[1]), c // grid[0] % grid[1], c % grid[0]], 1)
    want = O.voxelize_cells(pts, pts, coor, ok, max_points, max_voxels, 0)
    res = points_to_voxel_v2(pts, None, RANGE, SRANGE, None, max_points, max_voxels, resolution_HWD=grid,
                             coord_system="spherical", append_mode=0, cells=torch.tensor(cells))
    _compare(res, want)
    if max_voxels == 4000:
        assert want["voxel_num"] == np.unique(cells[ok]).size > 2500 and want["num_points_per_voxel"].max() == max_points


def test_every_point_in_one_cell():
    """70 000 points in a single cell: one segment, and the hash table's one slot takes every atomic."""
    n = 70000
    pts = np.random.default_rng(9).normal(0, 1, (n, 5)).astype(np.float32)
    cells = np.full(n, 37, np.int64)
    coor = np.tile(np.array([[0, 37 // 16, 37 % 16]]), (n, 1))
    want = O.voxelize_cells(pts, pts, coor, np.ones(n, bool), 7, 10, 0)
    res = points_to_voxel_v2(pts, None, RANGE, SRANGE, None, 7, 10, resolution_HWD=[16, 16, 4],
                             coord_system="spherical", append_mode=0, cells=torch.tensor(cells))
    _compare(res, want)
    assert want["voxel_num"] == 1 and want["num_points_per_voxel"][0] == 7


def test_small_and_degenerate_inputs():
    pts = np.array([[20, 1, 0.2, 0.5], [20, 1, 0.2, 0.6], [0, 0, 3, 0.1], [0, 0, 0, 0.2], [1e3, 5, 1, 0.3],
                    [30, -2, -1, 0.4], [20, 1, 0.2, 0.7]], np.float32)
    for mv in (1, 2, 5):
        res = points_to_voxel_v2(pts, None, RANGE, SRANGE, None, 2, mv, resolution_HWD=[8, 8, 4])
        want = O.points_to_voxel_v2(pts, RANGE, SRANGE, 2, mv, [8, 8, 4], "spherical")
        _compare(res, want)
    res = points_to_voxel_v2(np.zeros((0, 4), np.float32), None, RANGE, SRANGE, None, 2, 10, resolution_HWD=[8, 8, 4])
    assert res["voxel_num"] == 0 and float(res["voxels"].abs().sum()) == 0.0
    with pytest.raises(ValueError):
        points_to_voxel_v2(pts, None, RANGE, SRANGE, None, 2, 10, resolution_HWD=[8, 8, 4], coord_system="polar")


def test_voxelization_vfe_feeds_the_convolution():
    """datagen.VoxelizationVFE (reference test/common.py:30-59 builds its 'real' inputs with it):
    file -> mean voxel features + coordinates -> SparseConvTensor -> convolution."""
    shape_dwh = [16, 64, 64]
    vvfe = VoxelizationVFE(resolution_HWD=shape_dwh[::-1])
    voxels, coords = vvfe.generate(KITTI, torch.device("cuda:0"))
    pts = np.fromfile(KITTI, dtype=np.float32).reshape(-1, 4)
    want = O.points_to_voxel_v2(pts, RANGE, SRANGE, 2, 24000, shape_dwh[::-1], "spherical")
    m = want["voxel_num"]
    if voxels.shape[0] == m and np.array_equal(coords.cpu().numpy(), want["coordinates"][:m]):
        mean = O.simple_voxel(want["voxels"][:m], want["num_points_per_voxel"][:m])
        np.testing.assert_allclose(voxels.cpu().numpy(), mean, rtol=1e-6, atol=1e-7)
    assert abs(voxels.shape[0] - m) <= max(2, m // 500)
    assert (coords.cpu().numpy().max(0) < shape_dwh).all()
    batch = merge_batch_torch([{"voxels": voxels, "coordinates": coords}] * 2)
    assert batch["coordinates"].shape == (2 * voxels.shape[0], 4) and batch["coordinates"][:, 0].max() == 1
    x = sphconv.SparseConvTensor(batch["voxels"], shape_dwh, 2, indices=batch["coordinates"])
    y = sphconv.SubMConv3d(4, 8, 3).cuda()(x)
    assert y.feature.shape == (2 * voxels.shape[0], 8) and torch.isfinite(y.feature).all()


def test_sphere_branch_without_resolution():
    """points_to_voxel_v2 without resolution_HWD (voxelize.py:184-206) on the reference's scan against the
    oracle; the radial bounds are given in log r as the reference's C++ reads them (point2voxel.h:366)."""
    pts = np.fromfile(KITTI, dtype=np.float32).reshape(-1, 4)
    vs = [(np.log(70.4) - np.log(6.0)) / 64, 90.0 / 512, 12.5 / 64]
    srange = [float(np.log(6.0)), -45.0, 87.5, float(np.log(70.4)), 45.0, 100.0]
    want = O.points_to_voxel_sphere(pts, vs, srange, max_points=3, max_voxels=20000)
    assert want["grid_size"] == [64, 512, 64]
    got = points_to_voxel_v2(pts, vs, None, srange, None, max_points=3, max_voxels=20000, return_cells=True)
    # bins depend on float32 acos / asin / log: points within 1e-3 of a bin boundary may fall either way
    cells = got["cells"].cpu().numpy()
    x, y, z = pts[:, 0].astype(np.float64), pts[:, 1].astype(np.float64), pts[:, 2].astype(np.float64)
    r = np.sqrt(x * x + y * y + z * z)
    fb = np.stack([(np.log(r) - srange[0]) / vs[0], (np.degrees(np.arcsin(y / np.sqrt(x * x + y * y))) + 45.0) / vs[1],
                   (np.degrees(np.arccos(z / r)) - 87.5) / vs[2]], 1)
    near = (np.abs(fb - np.rint(fb)) < 1e-3).any(1)
    ok = np.isfinite(fb).all(1) & (fb >= 0).all(1) & (fb[:, 0] < 64) & (fb[:, 1] < 512) & (fb[:, 2] < 64)
    ref_cells = np.where(ok, (np.floor(fb[:, 2]) * 512 + np.floor(fb[:, 1])) * 64 + np.floor(fb[:, 0]), -1).astype(np.int64)
    assert near.mean() < 0.02 and np.array_equal(cells[~near], ref_cells[~near])
    if np.array_equal(cells, ref_cells):          # no point changed its bin: the whole result is the oracle's
        n = want["voxel_num"]
        assert got["voxel_num"] == n
        assert np.array_equal(got["coordinates"][:n].cpu().numpy(), want["coordinates"][:n])
        assert np.array_equal(got["voxels"][:n].cpu().numpy(), want["voxels"][:n])
        assert np.array_equal(got["num_points_per_voxel"][:n].cpu().numpy(), want["num_points_per_voxel"][:n])
    # the sequential rules on the GPU's own cells
    seq = O.voxelize_cells(pts, None, np.stack([cells // (512 * 64), (cells // 64) % 512, cells % 64], 1), cells >= 0, 3, 20000)
    n = seq["voxel_num"]
    assert got["voxel_num"] == n and n > 1000
    assert np.array_equal(got["coordinates"][:n].cpu().numpy(), seq["coordinates"][:n])
    assert np.array_equal(got["voxels"][:n].cpu().numpy(), seq["voxels"][:n])
    assert np.array_equal(got["num_points_per_voxel"][:n].cpu().numpy(), seq["num_points_per_voxel"][:n])
    # the generator class passes its missing resolution through
    gen = VoxelGeneratorV3(vs, [6, -40, -3, 70.4, 40, 1], srange, 3, 20000)
    assert gen.grid_size.tolist() == [64, 512, 64]
    res = gen.generate(pts)
    assert res["voxels"].shape[0] == n and np.array_equal(res["coordinates"].cpu().numpy(), seq["coordinates"][:n])
