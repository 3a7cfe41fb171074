"""Point cloud -> voxels on the GPU (reference: sphconv/utils/voxelize.py,
sphconv/utils/voxel_generator.py, sphconv/utils/coord_transform.py, include/point2voxel.h).

``points_to_voxel_v2`` keeps the reference's arguments and result dictionary
(voxelize.py:126-214); the coordinate transform, the binning and the voxel numbering in
order of first appearance run in one C call (``sph_points_to_voxel``)."""
import ctypes as C
from typing import List, Optional

import numpy as np
import torch

from . import _lib as L

COORD_SYSTEMS = {"spherical": 0, "l-spherical": 1, "cylinder": 2, "l-cylinder": 3, "hybrid": 4, "l-hybrid": 5}


def system_range(coors_range, sphere_coors_range, coord_system: str) -> np.ndarray:
    """Range of the system coordinates (c0, c1, c2), min then max: degrees become radians and
    logarithmic systems take the log of the radial bounds (coord_transform.py:18-23, 36-41,
    53-58, 70-75, 90-95, 110-115)."""
    v, s = [float(x) for x in coors_range], [float(x) for x in sphere_coors_range]
    rad = np.radians
    lo0, hi0 = (np.log(s[0]), np.log(s[3])) if coord_system.startswith("l-") else (s[0], s[3])
    if coord_system in ("cylinder", "l-cylinder"):
        return np.array([lo0, rad(s[1]), v[2], hi0, rad(s[4]), v[5]], dtype=np.float64)
    if coord_system in COORD_SYSTEMS:
        return np.array([lo0, rad(s[1]), rad(s[2]), hi0, rad(s[4]), rad(s[5])], dtype=np.float64)
    raise ValueError("unknown coord_system %r (one of %s)" % (coord_system, sorted(COORD_SYSTEMS)))


def points_to_voxel_v2(points, voxel_size, coors_range, sphere_coors_range, coor_to_voxelidx=None,
                       max_points=1, max_voxels=30000, pad_output=False,
                       resolution_HWD: Optional[List[int]] = None, coord_system: Optional[str] = None,
                       append_mode: int = 0, cells: Optional[torch.Tensor] = None, return_cells: bool = False):
    """voxelize.py:126-214.  ``points`` [N,>=4] float32 (numpy or
    torch) -> dict with ``voxels`` [max_voxels,max_points,W], ``coordinates`` [max_voxels,3] int32,
    ``num_points_per_voxel`` [max_voxels] int32, ``voxel_point_mask`` [max_voxels,max_points,1] (GPU
    tensors, zero beyond ``voxel_num``) and ``voxel_num`` (int; one 4-byte device->host read).
    ``coor_to_voxelidx`` (the reference's dense scratch map) is accepted and not used; ``voxel_size``
    only without ``resolution_HWD`` (then: log-spherical bins of that size, coordinates (theta, phi, r),
    and no appended columns are filled: point2voxel.h:387-390 copies the point as it is).
    ``cells`` [N] int64 overrides the computed cells; ``return_cells`` adds them as ``res["cells"]``."""
    f32 = np.float32
    if resolution_HWD is None:
        # voxelize.py:184-206 -> points_to_voxel_3d_sphere_np (point2voxel.h:316-399): bins of (log r,
        # phi, theta) from a voxel size (metres of log r, degrees, degrees) and sphere_coors_range taken
        # as it is (degrees -> radians; its radial bounds are used in the units of log r, :366); the
        # grid is round(range / voxel size) (:337-340), all in the points' float32
        vsz = np.asarray(voxel_size, dtype=np.float64)
        srg = np.asarray(sphere_coors_range, dtype=np.float64)
        vs = [f32(vsz[0]), f32(np.radians(vsz[1])), f32(np.radians(vsz[2]))]
        rng = np.array([srg[0], np.radians(srg[1]), np.radians(srg[2]), srg[3], np.radians(srg[4]), np.radians(srg[5])],
                       dtype=np.float64).astype(np.float32)
        grid = [int(np.floor(np.float64(f32(f32(rng[3 + i] - rng[i]) / vs[i])) + 0.5)) for i in range(3)]
        if min(grid) <= 0:
            raise L.SphconvError("voxel size %s leaves no cell in range %s" % (list(vsz), list(srg)))
        coord_system = "l-spherical"
        pad_cols, append_mode = (3 if append_mode == 1 else 0), 0
    else:
        pad_cols = 0
        coord_system = coord_system or "spherical"
        rng = system_range(coors_range, sphere_coors_range, coord_system).astype(np.float32)
        grid = [int(v) for v in resolution_HWD]
        # float32 voxel sizes, as the reference's float instantiation computes them (point2voxel.h:436-439)
        vs = [f32((rng[3 + i] - rng[i]) / f32(grid[i])) for i in range(3)]
    if isinstance(points, np.ndarray):
        points = torch.from_numpy(np.ascontiguousarray(points, dtype=np.float32))
    dev = points.device if points.is_cuda else torch.device("cuda", torch.cuda.current_device())
    pts = points.to(device=dev, dtype=torch.float32).contiguous()
    n, nfeat = pts.shape
    width = nfeat + 3 if append_mode == 1 else nfeat
    lib = L.lib()
    voxels = torch.empty((max_voxels, max_points, width), dtype=torch.float32, device=dev)
    mask = torch.empty((max_voxels, max_points), dtype=torch.float32, device=dev)
    coors = torch.empty((max_voxels, 3), dtype=torch.int32, device=dev)
    num = torch.empty((max_voxels,), dtype=torch.int32, device=dev)
    voxel_num = torch.empty(1, dtype=torch.int32, device=dev)
    nbytes = lib.sph_points_to_voxel_workspace(n, grid[0], grid[1], grid[2])
    if nbytes == 0:
        raise L.SphconvError("bad resolution %s, or more than 2^29 points (%d)" % (grid, n))
    work = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    cell_out = torch.empty(n, dtype=torch.int64, device=dev) if return_cells else None
    if cells is not None:
        cells = cells.to(device=dev, dtype=torch.int64).contiguous()
    with torch.cuda.device(dev):
        L.check(lib.sph_points_to_voxel(L.ptr(pts) if n else None, n, nfeat, COORD_SYSTEMS[coord_system],
                                        float(rng[0]), float(rng[1]), float(rng[2]), float(vs[0]), float(vs[1]),
                                        float(vs[2]), grid[0], grid[1], grid[2], int(max_points), int(max_voxels),
                                        int(append_mode), L.ptr(voxels), L.ptr(mask), L.ptr(coors), L.ptr(num),
                                        L.ptr(voxel_num), L.ptr(cells), L.ptr(cell_out), L.ptr(work), nbytes,
                                        L.stream()))
    if pad_cols:
        voxels = torch.nn.functional.pad(voxels, (0, pad_cols))
    res = {"voxels": voxels, "coordinates": coors, "num_points_per_voxel": num,
           "voxel_point_mask": mask.reshape(-1, max_points, 1), "voxel_num": int(voxel_num.item())}
    if return_cells:
        res["cells"] = cell_out
    return res


class VoxelGeneratorV3:
    """voxel_generator.py:6-97"""

    def __init__(self, voxel_size, point_cloud_range, point_cloud_sphere_range, max_num_points, max_voxels=30000,
                 resolution_HWD: List[int] = None, coord_system=None, append_mode=0):
        point_cloud_sphere_range = np.array(point_cloud_sphere_range, dtype=np.float32)
        point_cloud_range = np.array(point_cloud_range, dtype=np.float32)
        if resolution_HWD is not None:
            grid_size = np.array(resolution_HWD, dtype=np.int64)
        else:
            voxel_size = np.array(voxel_size, dtype=np.float32)
            grid_size = np.round((point_cloud_sphere_range[3:] - point_cloud_sphere_range[:3]) / voxel_size).astype(np.int64)
        self._voxel_size = voxel_size
        self._point_cloud_range = point_cloud_range
        self._point_cloud_sphere_range = point_cloud_sphere_range
        self._max_num_points = max_num_points
        self._max_voxels = max_voxels
        self._grid_size = grid_size
        self._resolution_HWD = resolution_HWD
        self._coord_system = coord_system
        self._append_mode = append_mode

    def generate(self, points, max_voxels=None):
        res = points_to_voxel_v2(points, self._voxel_size, self._point_cloud_range, self._point_cloud_sphere_range,
                                 None, self._max_num_points, max_voxels or self._max_voxels,
                                 resolution_HWD=self._resolution_HWD,
                                 coord_system=self._coord_system, append_mode=self._append_mode)
        for k, v in res.items():
            if k != "voxel_num":
                res[k] = v[:res["voxel_num"]]
        return res

    @property
    def voxel_size(self):
        return self._voxel_size

    @property
    def max_num_points_per_voxel(self):
        return self._max_num_points

    @property
    def point_cloud_range(self):
        return self._point_cloud_range

    @property
    def grid_size(self):
        return self._grid_size
