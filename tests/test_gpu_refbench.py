"""The reference author's own benchmark shapes (reference test/bench_conv.py:131-133: batch 8, 64 -> 64, grid
[64, 512, 512], 3x3x3 stride 2 padding 1; test/Untitled.ipynb cell 1: batch 3, submanifold, same grid) at full
size: rules bit-exact and the fp16 forward within tolerance against the C oracle.  The compressed axis has 512
bins here (256 on the strided output), so this is the one workload that takes the paths for more than 64 bins
everywhere (several passes of bin masks per output column, the general fiber join) at size.

Inputs as in the reference (test/common.py:30-59): KITTI scans voxelised on a spherical 512 x 512 x 64 grid
(two points per voxel, mean VFE), channels repeated from 4 to 64.  The reference cycles through its four scans;
here every sample is the one committed scan (the reference's test/000000.bin) turned by two more degrees
about the vertical axis."""
import os

import numpy as np
import pytest
import torch

import helpers as H
import gpu_helpers as G
from oracle import oracle as O
import sphconv_amd as sphconv
from sphconv_amd import sphconv_cuda as ext
from sphconv_amd.rulebook import RuleBook
from sphconv_amd.synth import lidar_scan_batch

pytestmark = pytest.mark.gpu
KITTI = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kitti_000000_reduced.bin")
SHAPE = [64, 512, 512]


def refbench_inputs(batch, channels=64):
    """-> (feature [N,channels] fp16 on the GPU, indices [N,4] int32 (b, d, w, h))"""
    pts = np.fromfile(KITTI, dtype=np.float32).reshape(-1, 4)
    return lidar_scan_batch(pts, batch, SHAPE, channels, G.DEV)


@pytest.mark.parametrize("subm,batch", [(False, 8), (True, 3)], ids=["k3s2p1-b8", "subm-b3"])
def test_reference_benchmark_shape(subm, batch):
    feature, indices = refbench_inputs(batch)
    x = sphconv.SparseConvTensor(feature, SHAPE, batch, indices=indices)
    n = int(x.feature.shape[0])
    assert n > 10000 * batch
    z_idx, z_ptr = x.z_idx.cpu().numpy(), x.z_ptr.cpu().numpy()
    kernel, stride, padding = [3, 3, 3], ([1, 1, 1] if subm else [2, 2, 2]), [1, 1, 1]
    if subm:
        oshape = SHAPE
        book = RuleBook.build_subm(x.z_idx, x.z_ptr, batch, SHAPE, kernel)
        ora = O.get_rules_subm(z_idx, z_ptr, batch, SHAPE, oshape, kernel, stride, padding, n_max=256)
    else:
        oshape = H.out_shape_of(SHAPE, kernel, stride, padding)
        assert oshape == [32, 256, 256]
        book = RuleBook.build(x.z_idx, x.z_ptr, batch, SHAPE, oshape, kernel, stride, padding)
        ora = O.get_rules(z_idx, z_ptr, batch, SHAPE, oshape, kernel, stride, padding, n_max=512)
    oz_idx, oz_ptr, rules, rule_size, dropped = ora
    assert dropped == 0
    m = int(oz_idx.shape[0])
    assert book.out_rows == m
    assert np.array_equal(book.oz_idx.cpu().numpy(), oz_idx) and np.array_equal(book.oz_ptr.cpu().numpy(), oz_ptr)
    assert np.array_equal(G.book_triples(book.fwd), G.oracle_triples(rules, rule_size))
    assert np.array_equal(G.book_triples(book.transposed()), G.oracle_triples(rules, rule_size, swap=True))
    rng = np.random.default_rng(7)
    w = torch.tensor((rng.standard_normal((27, 64, 64)) / np.sqrt(27 * 64)).astype(np.float32)).half()
    out = ext.rule_conv(x.feature, w.to(G.DEV), book, None, m)
    want = O.rule_conv(x.feature.float().cpu().numpy(), w.float().numpy(), rules, rule_size, m)
    got = out.float().cpu().numpy()
    assert np.abs(want).mean() > 1e-3
    # fp16 storage, fp32 accumulate: one rounding of the fp32 sum (north_star: rtol 1e-2, atol 1e-3)
    assert (np.abs(got - want) <= 2.0 ** -10 * np.abs(want) + 1e-3).all()
