"""Pins the CPU oracle's tensor construction and rule generation (no GPU).

Checks, none of which reuse the oracle's code:
  * brute-force enumeration of the pair definition with Python dicts on every
    literal coordinate list / parameter tuple the reference's tests hold
    (tests/golden/ref_cases.json; reference test_rules.py:158-406, test_conv.py:119-363);
  * the reference's own torch check: active output set == conv3d(occ, ones) != 0
    (reference test_rules.py:14-60);
  * closed forms and invariants (tile_n_max, out_spatial, centre offset count,
    pair symmetry, pair count == conv3d(occ, ones) summed at active sites).
"""
import numpy as np
import pytest
import torch

import helpers as H
from oracle import oracle as O

CASES = H.load_ref_cases()


def _rule_calls():
    out = []
    for t in CASES:
        if t["file"] not in ("test/test_rules.py", "test/test_conv.py", "test/test_module.py"):
            continue
        for c in t["calls"]:
            a = c["args"]
            if "spatial_shape_DWH" not in a and t["file"] != "test/test_rules.py":
                continue
            out.append(pytest.param(t["tensors"][c["coords"]], a,
                                    id="%s:%d" % (t["file"].split("/")[-1], c["line"])))
    return out


def _params(a):
    subm = bool(a.get("subm", False))
    B = a.get("batch_size", 1)
    shape = a.get("spatial_shape_DWH", [8, 8, 8])
    kernel = a.get("kernel_size", [3, 3, 3])
    stride = a.get("stride", [2, 2, 2])
    padding = a.get("padding", [1, 1, 1])
    if subm:
        padding = [k // 2 for k in kernel]
        stride = [1, 1, 1]
    return subm, B, shape, kernel, stride, padding


@pytest.mark.parametrize("coords,args", _rule_calls())
def test_rules_match_bruteforce(coords, args):
    subm, B, shape, kernel, stride, padding = _params(args)
    idx = H.dup_with_batch_idx(coords, B)
    rng = np.random.default_rng(0)
    idx = idx[rng.permutation(idx.shape[0])]          # COO order must not matter
    feat = rng.standard_normal((idx.shape[0], 3)).astype(np.float32)

    # init_tensor vs numpy
    sidx, z_idx_np, z_ptr_np, order = H.csr_from_indices(idx, B, shape)
    f2, z_idx, z_ptr, perm = O.init_tensor(feat, idx, B, shape)
    assert np.array_equal(z_idx, z_idx_np) and np.array_equal(z_ptr, z_ptr_np)
    assert np.array_equal(f2, feat[order])
    assert np.array_equal(f2[perm], feat)

    oshape = list(shape) if subm else O.out_spatial(shape, kernel, stride, padding)
    assert oshape == (list(shape) if subm else H.out_shape_of(shape, kernel, stride, padding))
    if min(oshape) <= 0:
        pytest.skip("empty output grid")
    fn = O.get_rules_subm if subm else O.get_rules
    oz_idx, oz_ptr, rules, rule_size, dropped = fn(z_idx, z_ptr, B, shape, oshape, kernel,
                                                   stride, padding, (1, 1, 1), (2, 2))
    assert dropped == 0
    out_coords, pairs, oshape_b = H.brute_rules(sidx, B, shape, kernel, stride, padding, subm)
    assert oshape_b == oshape
    assert H.rules_to_dict(rules, rule_size) == pairs
    # unused slots keep the -1 fill
    for t, k in zip(*np.nonzero(rule_size >= 0)):
        assert (rules[t, k, :, rule_size[t, k]:] == -1).all()

    # output coordinates: rows numbered by (b,o0,o1,o2) ascending
    assert oz_idx.shape[0] == out_coords.shape[0]
    assert np.array_equal(oz_idx, out_coords[:, 3])
    col = (out_coords[:, 0].astype(np.int64) * oshape[0] + out_coords[:, 1]) * oshape[1] + out_coords[:, 2]
    cnt = np.bincount(col, minlength=B * oshape[0] * oshape[1])
    assert np.array_equal(np.asarray(oz_ptr).ravel(), np.cumsum(cnt))

    # the reference's torch check (test_rules.py:51-60): active set == conv3d(occ, ones) != 0
    occ = H.dense_from_rows(np.ones((sidx.shape[0], 1)), sidx, B, shape)
    ones_w = np.ones((*kernel, 1, 1))
    hits = H.dense_conv(occ, ones_w, stride, padding, oshape)
    if not subm:
        act = H.dense_from_rows(np.ones((out_coords.shape[0], 1)), out_coords, B, oshape)
        assert torch.equal(act != 0, hits != 0)
        assert int(rule_size.sum()) == int(hits.sum().item())
    else:
        assert int(rule_size.sum()) == int(H.gather_rows(hits, sidx).sum().item())
        kv = int(np.prod(kernel))
        if all(k % 2 == 1 for k in kernel):
            centre = kv // 2
            assert int(rule_size[:, centre].sum()) == sidx.shape[0]
            # pair (i,j) at k  <=>  pair (j,i) at KV-1-k
            per_k = {}
            for (t, k), lst in pairs.items():
                per_k.setdefault(k, set()).update(lst)
            for k, s in per_k.items():
                assert {(j, i) for i, j in s} == per_k.get(kv - 1 - k, set())
    # per-k output rows unique; every pair's tile is the tile of its output column
    tgw = -(-oshape[1] // 2)
    for (t, k), lst in H.rules_to_dict(rules, rule_size).items():
        outs = [j for _, j in lst]
        assert len(set(outs)) == len(outs)
        for _, j in lst:
            assert t == (out_coords[j, 1] // 2) * tgw + out_coords[j, 2] // 2


def test_closed_forms():
    # rules.cu:21-28 evaluated by hand: B=1, inT=4x4, S=[64,512,32], NNZ=39256
    # sparsity = 39256/1048576; size = 16*32*sparsity*2 = 38.33..; (int)(102.33) & ~15 = 96
    assert O.tile_n_max(1, [64, 512, 32], [3, 3, 3], [1, 1, 1], [2, 2], 39256) == 96
    # stride 2: inT = 2*(2-1)+3 = 5
    assert O.lib().orc_in_tile_size(2, 2, 3) == 5
    for i, k, s, p in [(8, 3, 2, 1), (9, 3, 2, 1), (64, 3, 2, 1), (2, 2, 1, 1), (3, 2, 2, 0), (20, 3, 1, 0)]:
        ref = torch.nn.functional.conv1d(torch.zeros(1, 1, i), torch.zeros(1, 1, k), None, s, p).shape[-1]
        assert O.out_spatial([i] * 3, [k] * 3, [s] * 3, [p] * 3) == [ref] * 3


def test_overflow_is_reported():
    # a full 4x4x8 block with tile_n_max forced to 16 must drop pairs, and say so
    coords = np.array([[0, a, b, c] for a in range(4) for b in range(4) for c in range(8)], np.int32)
    _, z_idx, z_ptr, _ = H.csr_from_indices(coords, 1, [4, 4, 8])
    *_, rules, rule_size, dropped = O.get_rules_subm(z_idx, z_ptr, 1, [4, 4, 8], [4, 4, 8],
                                                      [3, 3, 3], [1, 1, 1], [1, 1, 1], n_max=16)
    assert dropped > 0 and rule_size.max() > 16


@pytest.mark.parametrize("seed", [0, 1])
@pytest.mark.parametrize("subm", [True, False])
def test_random_grid_vs_bruteforce(seed, subm):
    rng = np.random.default_rng(seed)
    B, shape = 2, [7, 9, 12]
    occ = rng.random((B, *shape)) < 0.15
    idx = np.argwhere(occ).astype(np.int32)
    sidx, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    kernel, stride, padding = ([3, 3, 3], [1, 1, 1], [1, 1, 1]) if subm else ([3, 2, 3], [2, 1, 2], [1, 0, 1])
    oshape = shape if subm else H.out_shape_of(shape, kernel, stride, padding)
    fn = O.get_rules_subm if subm else O.get_rules
    for tile in [(2, 2), (3, 4), (1, 64)]:
        oz_idx, oz_ptr, rules, rule_size, dropped = fn(z_idx, z_ptr, B, shape, oshape, kernel,
                                                       stride, padding, (1, 1, 1), tile, n_max=512)
        out_coords, pairs, _ = H.brute_rules(sidx, B, shape, kernel, stride, padding, subm, tile)
        assert dropped == 0
        assert H.rules_to_dict(rules, rule_size) == pairs
        assert np.array_equal(oz_idx, out_coords[:, 3])
