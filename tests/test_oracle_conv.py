"""Pins the CPU oracle's convolution (forward, dgrad, wgrad, int8) without a GPU.

Independent references: torch dense conv3d in float64 (weight mapped by
permute(4,3,0,1,2) as reference test_grad.py:31 does), torch autograd through it
(pattern of reference test_grad.py:7-36), exact int64 numpy for int8, and special
cases that reduce to closed forms (K=1 -> feature @ W[0]; all-ones -> iC * #neighbours).
"""
import numpy as np
import pytest
import torch

import helpers as H
from oracle import oracle as O

CASES = H.load_ref_cases()


def _conv_calls():
    out = []
    for t in CASES:
        if t["file"] != "test/test_conv.py":
            continue
        for c in t["calls"]:
            out.append(pytest.param(t["tensors"][c["coords"]], c["args"],
                                    id="test_conv.py:%d" % c["line"]))
    return out


def _setup(coords, B, shape, kernel, stride, padding, subm, ic, oc, seed=0, tile=(2, 2)):
    rng = np.random.default_rng(seed)
    idx = H.dup_with_batch_idx(coords, B)
    sidx, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    if subm:
        padding = [k // 2 for k in kernel]
    oshape = list(shape) if subm else H.out_shape_of(shape, kernel, stride, padding)
    fn = O.get_rules_subm if subm else O.get_rules
    oz_idx, oz_ptr, rules, rule_size, dropped = fn(z_idx, z_ptr, B, shape, oshape, kernel, stride,
                                                   padding, (1, 1, 1), tile)
    assert dropped == 0
    out_coords, _, _ = H.brute_rules(sidx, B, shape, kernel, stride, padding, subm, tile)
    feat = rng.standard_normal((sidx.shape[0], ic)).astype(np.float32)
    w = (rng.standard_normal((*kernel, ic, oc)) / np.sqrt(np.prod(kernel) * ic)).astype(np.float32)
    return dict(sidx=sidx, out_coords=out_coords, oshape=oshape, rules=rules, rule_size=rule_size,
                feat=feat, w=w, padding=padding, tile=tile, B=B, shape=shape, kernel=kernel,
                stride=stride)


def _dense_forward(s, feat=None, w=None, dtype=torch.float64):
    feat = s["feat"] if feat is None else feat
    w = s["w"] if w is None else w
    dense = H.dense_from_rows(feat, s["sidx"], s["B"], s["shape"], dtype)
    y = H.dense_conv(dense, w, s["stride"], s["padding"], s["oshape"])
    return H.gather_rows(y, s["out_coords"]).numpy()


@pytest.mark.parametrize("coords,args", _conv_calls())
def test_forward_vs_dense_conv3d(coords, args):
    a = args
    s = _setup(coords, a["batch_size"], a["spatial_shape_DWH"], a["kernel_size"], a["stride"],
               a["padding"], a.get("subm", False), a["in_channels"], a["out_channels"])
    kv = int(np.prod(a["kernel_size"]))
    out = O.rule_conv(s["feat"], s["w"].reshape(kv, a["in_channels"], a["out_channels"]),
                      s["rules"], s["rule_size"], s["out_coords"].shape[0])
    ref = _dense_forward(s)
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-5)


GRID = [(0, True, [3, 3, 3], [1, 1, 1], [1, 1, 1], 16, 16),
        (1, False, [3, 3, 3], [2, 2, 2], [1, 1, 1], 8, 24),
        (2, False, [2, 3, 1], [1, 2, 1], [0, 1, 0], 5, 7),
        (3, True, [1, 1, 1], [1, 1, 1], [0, 0, 0], 12, 4)]


def _random_case(seed, subm, kernel, stride, padding, ic, oc, tile=(2, 2)):
    rng = np.random.default_rng(seed)
    B, shape = 2, [6, 10, 9]
    occ = rng.random((B, *shape)) < 0.2
    idx = np.argwhere(occ).astype(np.int32)
    return _setup(idx, B, shape, kernel, stride, padding, subm, ic, oc, seed, tile)


@pytest.mark.parametrize("seed,subm,kernel,stride,padding,ic,oc", GRID)
def test_forward_backward_vs_autograd(seed, subm, kernel, stride, padding, ic, oc):
    s = _random_case(seed, subm, kernel, stride, padding, ic, oc)
    kv = int(np.prod(kernel))
    w3 = s["w"].reshape(kv, ic, oc)
    M = s["out_coords"].shape[0]
    out = O.rule_conv(s["feat"], w3, s["rules"], s["rule_size"], M)

    # float64 autograd through the dense conv, gathered at active sites
    f_t = torch.tensor(s["feat"], dtype=torch.float64, requires_grad=True)
    w_t = torch.tensor(s["w"], dtype=torch.float64, requires_grad=True)
    c_in = torch.as_tensor(s["sidx"], dtype=torch.long)
    dense = torch.zeros((s["B"], *s["shape"], ic), dtype=torch.float64)
    dense = dense.index_put((c_in[:, 0], c_in[:, 1], c_in[:, 2], c_in[:, 3]), f_t)
    dense = dense.permute(0, 4, 1, 2, 3)
    y = torch.nn.functional.conv3d(dense, w_t.permute(4, 3, 0, 1, 2), None, tuple(stride),
                                   tuple(s["padding"]))
    y = y[:, :, :s["oshape"][0], :s["oshape"][1], :s["oshape"][2]]
    c_out = torch.as_tensor(s["out_coords"], dtype=torch.long)
    y_rows = y[c_out[:, 0], :, c_out[:, 1], c_out[:, 2], c_out[:, 3]]
    g = np.random.default_rng(seed + 100).standard_normal((M, oc)).astype(np.float32)
    (y_rows * torch.tensor(g, dtype=torch.float64)).sum().backward()

    np.testing.assert_allclose(out, y_rows.detach().numpy(), rtol=1e-5, atol=1e-5)
    tgs = [-(-s["oshape"][0] // 2), -(-s["oshape"][1] // 2)]
    w_perm = np.ascontiguousarray(w3.transpose(0, 2, 1))         # functional.py:73
    d_feat, d_w = O.rule_conv_backward(g, s["feat"], w_perm, s["rules"], s["rule_size"], tgs)
    np.testing.assert_allclose(d_feat, f_t.grad.numpy(), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(d_w, w_t.grad.numpy().reshape(kv, ic, oc), rtol=1e-5, atol=2e-5)


def test_k1_reduces_to_matmul():
    s = _random_case(5, True, [1, 1, 1], [1, 1, 1], [0, 0, 0], 9, 6)
    out = O.rule_conv(s["feat"], s["w"].reshape(1, 9, 6), s["rules"], s["rule_size"],
                      s["sidx"].shape[0])
    np.testing.assert_allclose(out, s["feat"].astype(np.float64) @ s["w"].reshape(9, 6), rtol=1e-5,
                               atol=1e-6)


def test_all_ones_counts_neighbours():
    s = _random_case(6, True, [3, 3, 3], [1, 1, 1], [1, 1, 1], 4, 3)
    n = s["sidx"].shape[0]
    out = O.rule_conv(np.ones((n, 4), np.float32), np.ones((27, 4, 3), np.float32), s["rules"],
                      s["rule_size"], n)
    occ = H.dense_from_rows(np.ones((n, 1)), s["sidx"], s["B"], s["shape"])
    nb = H.gather_rows(H.dense_conv(occ, np.ones((3, 3, 3, 1, 1)), [1, 1, 1], [1, 1, 1], s["shape"]),
                       s["sidx"]).numpy()
    assert np.array_equal(out, np.repeat(4.0 * nb, 3, axis=1).astype(np.float32))


def test_tile_size_does_not_change_results():
    a = _random_case(7, False, [3, 3, 3], [2, 2, 2], [1, 1, 1], 8, 8, tile=(2, 2))
    b = _random_case(7, False, [3, 3, 3], [2, 2, 2], [1, 1, 1], 8, 8, tile=(1, 5))
    M = a["out_coords"].shape[0]
    oa = O.rule_conv(a["feat"], a["w"].reshape(27, 8, 8), a["rules"], a["rule_size"], M)
    ob = O.rule_conv(b["feat"], b["w"].reshape(27, 8, 8), b["rules"], b["rule_size"], M)
    np.testing.assert_allclose(oa, ob, rtol=1e-5, atol=1e-6)


def test_stable_case_extreme_weights():
    """The reference's test_stable.py case: 74 voxels on [6,6,20], stride 2, 64->64,
    features all 100 with rows 0 and 3 set to 8 and 16, weights randn/2 with planes
    set to 8, 100 and 1/64 (test_stable.py:108-110,154-158).  Oracle: dense conv3d, fp64."""
    t = [c for c in CASES if c["file"] == "test/test_stable.py"][0]
    coords = np.array(t["tensors"]["indices_bzyx"], np.int32)
    s = _setup(coords, 1, [6, 6, 20], [3, 3, 3], [2, 2, 2], [1, 1, 1], False, 64, 64)
    # features are assigned in the COO order of the reference's list
    raw = np.full((coords.shape[0], 64), 100.0, np.float32)
    raw[0, :] = 8.0
    raw[3, :] = 16.0
    _, order = H.canonical_rows(coords)
    feat = raw[order]
    w = (np.random.default_rng(0).standard_normal((3, 3, 3, 64, 64)) / 2).astype(np.float32)
    w[1] = 8.0
    w[-1] = 100.0
    w[1, 2, 0, :5, :] = 1 / 64
    out = O.rule_conv(feat, w.reshape(27, 64, 64), s["rules"], s["rule_size"],
                      s["out_coords"].shape[0])
    ref = _dense_forward(s, feat, w)
    np.testing.assert_allclose(out, ref, rtol=1e-4, atol=1e-2)


def test_int8_exact():
    s = _random_case(8, True, [3, 3, 3], [1, 1, 1], [1, 1, 1], 16, 8)
    rng = np.random.default_rng(8)
    n = s["sidx"].shape[0]
    f8 = rng.integers(-128, 128, (n, 16), dtype=np.int8)
    w8 = rng.integers(-128, 128, (27, 16, 8), dtype=np.int8)
    scale = (rng.random(8).astype(np.float32) + 0.5) / 600.0
    q, acc = O.rule_conv_i8(f8, w8, scale, s["rules"], s["rule_size"], n, return_acc=True)
    # exact integer pair-sum from the brute-force pair list
    _, pairs, _ = H.brute_rules(s["sidx"], s["B"], s["shape"], [3, 3, 3], [1, 1, 1], [1, 1, 1], True)
    ref = np.zeros((n, 8), np.int64)
    for (t, k), lst in pairs.items():
        for i, j in lst:
            ref[j] += f8[i].astype(np.int64) @ w8[k].astype(np.int64)
    assert np.array_equal(acc, ref)
    # requantisation rule, restated with numpy float32 ops (IEEE, round-half-even)
    prod = ref.astype(np.int32).astype(np.float32) * scale[None, :]
    qref = np.clip(np.rint(prod), -128, 127).astype(np.int8)
    assert np.array_equal(q, qref)
    assert q.min() == -128 and q.max() == 127     # the case reaches saturation
