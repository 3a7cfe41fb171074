"""Seeded synthetic range-voxel generators for the benchmark configurations.

No reference counterpart: the reference's inputs come from KITTI files
(sphconv/data.py, test/common.py:30-59).  These generators produce LiDAR-like
occupancy directly in the per-column compressed layout the reference uses
(tensor.py:33-102): ``z_ptr [B,S0,S1]`` inclusive prefix sums of per-column
voxel counts and ``z_idx [N]`` the S2 (depth-bin) coordinate of each row,
fibers sorted ascending.

Axis names: S0 = rows of the range image, S1 = azimuth, S2 = depth bins.
In the Python API's terms ``spatial_shape_DWH = [S0, S1, S2]``.
"""
from typing import Tuple

import numpy as np


def _csr_from_occupancy(occ: np.ndarray) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """occ: bool [B,S0,S1,S2] -> (indices [N,4] int32 sorted, z_idx [N], z_ptr [B,S0,S1])."""
    B, S0, S1, S2 = occ.shape
    idx = np.argwhere(occ).astype(np.int32)              # lexicographic (b,s0,s1,s2)
    counts = occ.reshape(B * S0 * S1, S2).sum(axis=1)
    z_ptr = np.cumsum(counts, dtype=np.int64).astype(np.int32).reshape(B, S0, S1)
    z_idx = np.ascontiguousarray(idx[:, 3])
    return idx, z_idx, z_ptr


def occupancy_g1(B: int, S0: int, S1: int, S2: int, p: float = 0.6, seed: int = 0) -> np.ndarray:
    """Generator G1: each (b,s0,s1) column is occupied with probability ``p``;
    an occupied column holds 1..3 active bins (uniform count), distinct, uniform
    in [0,S2).  Sample ``b`` uses an independent stream derived from seed+b."""
    occ = np.zeros((B, S0, S1, S2), dtype=bool)
    for b in range(B):
        rng = np.random.default_rng(seed + b)
        col = rng.random((S0, S1)) < p
        cnt = rng.integers(1, 4, size=(S0, S1))
        cnt = np.minimum(cnt, S2)
        # three distinct uniform bins by sequential sampling without replacement
        b1 = rng.integers(0, S2, size=(S0, S1))
        b2 = rng.integers(0, max(S2 - 1, 1), size=(S0, S1))
        b2 = b2 + (b2 >= b1)
        lo, hi = np.minimum(b1, b2), np.maximum(b1, b2)
        b3 = rng.integers(0, max(S2 - 2, 1), size=(S0, S1))
        b3 = b3 + (b3 >= lo)
        b3 = b3 + (b3 >= hi)
        for j, bins in enumerate((b1, b2, b3)):
            s0i, s1i = np.nonzero(col & (cnt > j))
            occ[b, s0i, s1i, bins[s0i, s1i]] = True
    return occ


def occupancy_g2(B: int, S0: int, S1: int, S2: int, p: float = 0.5, seed: int = 0) -> np.ndarray:
    """Generator G2: column occupancy ``p``; each occupied column has 1..2 bins
    clustered around a smooth range profile
    ``bin = clamp(round(40 + 15 sin(2 pi s1 / S1) + N(0,3)), 0, S2-1)``
    (profile constants scaled by S2/64), duplicates merged."""
    occ = np.zeros((B, S0, S1, S2), dtype=bool)
    scale = S2 / 64.0
    w = np.arange(S1)
    for b in range(B):
        rng = np.random.default_rng(seed + b)
        col = rng.random((S0, S1)) < p
        cnt = rng.integers(1, 3, size=(S0, S1))
        prof = (40.0 + 15.0 * np.sin(w * 2.0 * np.pi / S1)) * scale
        for j in range(2):
            bins = np.rint(prof[None, :] + rng.normal(0.0, 3.0 * scale, size=(S0, S1)))
            bins = np.clip(bins, 0, S2 - 1).astype(np.int64)
            use = col & (cnt > j)
            s0i, s1i = np.nonzero(use)
            occ[b, s0i, s1i, bins[s0i, s1i]] = True
    return occ


def make_config(cfg: int, seed: int = 0, batch: int = None, p: float = None):
    """Occupancy of benchmark configuration ``cfg`` (1..5) -> dict with
    ``indices`` [N,4] (b,s0,s1,s2) int32, ``z_idx``, ``z_ptr`` and
    ``spatial_shape`` = [S0,S1,S2], ``batch``.  ``p`` overrides the generator's column occupancy
    (0.6 for G1, 0.5 for G2), e.g. to reach a given number of voxels."""
    if cfg == 1:
        B, shape, gen = 1, (64, 512, 32), occupancy_g1
    elif cfg == 2:
        B, shape, gen = 1, (64, 2048, 64), occupancy_g2
    elif cfg in (3, 4):
        B, shape, gen = 4, (64, 2048, 64), occupancy_g1
    elif cfg == 5:
        B, shape, gen = 8, (64, 512, 32), occupancy_g1
    else:
        raise ValueError("cfg must be 1..5")
    if batch is not None:
        B = batch
    occ = gen(B, *shape, seed=seed) if p is None else gen(B, *shape, p=p, seed=seed)
    idx, z_idx, z_ptr = _csr_from_occupancy(occ)
    return {"indices": idx, "z_idx": z_idx, "z_ptr": z_ptr,
            "spatial_shape": list(shape), "batch": B}


def config2_with_voxels(voxels: int, seed: int = 0):
    """Configuration 2's generator with its column occupancy raised (or lowered) until the scan holds about
    ``voxels`` active voxels (within 0.5 %): -> (dict as make_config, occupancy used)."""
    p = 0.5
    d = make_config(2, seed=seed, p=p)
    for _ in range(6):
        n = int(d["z_idx"].shape[0])
        if abs(n - voxels) <= 0.005 * voxels:
            break
        p = min(max(p * voxels / max(n, 1), 0.01), 1.0)
        d = make_config(2, seed=seed, p=p)
    return d, p


def lidar_scan_batch(points, batch: int, shape_dwh=(64, 512, 512), channels: int = 64, device="cuda:0"):
    """The reference's benchmark inputs (test/common.py:30-59, used by test/bench_conv.py:131-133): LiDAR scans
    voxelised on a spherical grid of ``shape_dwh`` cells (two points per voxel, at most 24000 voxels, mean VFE),
    merged into a batch, the four point channels repeated up to ``channels``.  ``points`` [m,4] float32 is ONE
    scan; sample i of the batch is that scan turned by 2 i degrees about the vertical axis (the reference
    cycles through four scan files).  -> (feature [N,channels] fp16, indices [N,4] int32 (b, d, w, h)) on
    ``device``."""
    import torch

    from .datagen import merge_batch_torch
    from .vfe import SimpleVoxel
    from .voxelize import VoxelGeneratorV3
    points = np.asarray(points, dtype=np.float32).reshape(-1, 4)
    gen = VoxelGeneratorV3(None, [6, -40, -3, 70.4, 40, 1], [6, -45, 87.5, 70.4, 45, 100], 2, 24000,
                           list(shape_dwh)[::-1], coord_system="spherical")
    vfe = SimpleVoxel(4)
    examples = []
    for i in range(batch):
        a = np.deg2rad(2.0 * i)
        rot = points.copy()
        rot[:, 0] = np.cos(a) * points[:, 0] - np.sin(a) * points[:, 1]
        rot[:, 1] = np.sin(a) * points[:, 0] + np.cos(a) * points[:, 1]
        res = gen.generate(torch.from_numpy(rot).to(device))
        voxels = vfe(res["voxels"], res["num_points_per_voxel"], res["coordinates"])
        examples.append({"voxels": voxels, "coordinates": res["coordinates"]})
    ex = merge_batch_torch(examples)
    feature = ex["voxels"].repeat((1, (channels + 3) // 4))[:, :channels]
    return feature.half().contiguous(), ex["coordinates"].int().contiguous()


def encoder_stack(in_channels: int = 16, widths=(16, 32, 64, 64), seed: int = 0, neighbours: float = 8.0):
    """The four-stage middle encoder of benchmark configuration 4 as a ``Sequential``:
    per stage two submanifold 3x3x3 convolutions sharing one rule book, then a 3x3x3
    convolution of stride 2 / padding 1, each followed by BatchNorm1d (evaluation mode,
    random affine and statistics) and ReLU.  Weights are normal with the variance that keeps
    activations of a voxel with ``neighbours`` active neighbours at unit scale."""
    import torch
    from torch import nn

    from .conv import SparseConv3d, SubMConv3d
    from .modules import Sequential

    gen = torch.Generator().manual_seed(seed)
    layers = []
    c_in = in_channels
    for s, c in enumerate(widths):
        for conv in (SubMConv3d(c_in, c, 3, indice_key="subm%d" % s), SubMConv3d(c, c, 3, indice_key="subm%d" % s),
                     SparseConv3d(c, c, 3, stride=2, padding=1)):
            with torch.no_grad():
                std = (2.0 / (neighbours * conv.in_channels)) ** 0.5
                conv.weight.copy_(torch.randn(conv.weight.shape, generator=gen) * std)
            bn = nn.BatchNorm1d(c)
            with torch.no_grad():
                bn.weight.copy_(0.75 + 0.5 * torch.rand(c, generator=gen))
                bn.bias.copy_(0.1 * torch.randn(c, generator=gen))
                bn.running_mean.copy_(0.1 * torch.randn(c, generator=gen))
                bn.running_var.copy_(0.75 + 0.5 * torch.rand(c, generator=gen))
            layers += [conv, bn, nn.ReLU()]
        c_in = c
    return Sequential(*layers).eval()
