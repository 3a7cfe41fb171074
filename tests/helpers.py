"""Independent checkers used to pin the oracle and the HIP path.

Nothing here shares code with oracle/sphconv_oracle.c: rules are enumerated
from the pair definition with Python dicts, convolution values come from
torch's dense conv3d in float64.
"""
import json
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def load_ref_cases():
    with open(os.path.join(HERE, "golden", "ref_cases.json")) as f:
        return json.load(f)


def dup_with_batch_idx(coords_zyx, batch_size):
    """[n,3] -> [n*B,4] with a leading batch column (what the reference's
    test/common.py dup_with_batch_idx does to its literal lists)."""
    c = np.asarray(coords_zyx, dtype=np.int32)
    if c.shape[1] == 4:
        return c
    out = [np.concatenate([np.full((c.shape[0], 1), b, np.int32), c], axis=1)
           for b in range(batch_size)]
    return np.concatenate(out, axis=0)


def canonical_rows(indices):
    """Sort COO rows lexicographically by (b,s0,s1,s2) -> (sorted indices, order)."""
    idx = np.asarray(indices, dtype=np.int64)
    order = np.lexsort((idx[:, 3], idx[:, 2], idx[:, 1], idx[:, 0]))
    return idx[order].astype(np.int32), order


def csr_from_indices(indices, B, shape):
    """Canonical (S2-sorted) per-column compressed form, by numpy only."""
    idx, order = canonical_rows(indices)
    S0, S1, S2 = shape
    col = (idx[:, 0].astype(np.int64) * S0 + idx[:, 1]) * S1 + idx[:, 2]
    counts = np.bincount(col, minlength=B * S0 * S1)
    z_ptr = np.cumsum(counts).astype(np.int32).reshape(B, S0, S1)
    return idx, idx[:, 3].copy(), z_ptr, order


def out_shape_of(shape, kernel, stride, padding, dilation=(1, 1, 1)):
    return [(i + 2 * p - d * (k - 1) - 1) // s + 1
            for i, k, s, p, d in zip(shape, kernel, stride, padding, dilation)]


def brute_rules(indices_sorted, B, shape, kernel, stride, padding, subm, tile=(2, 2)):
    """Enumerate pairs from the definition: input x pairs with output
    o_d = (x_d + pad_d - k_d)/s_d iff divisible and 0 <= o_d < O_d.
    Returns (out_coords sorted [M,4], pairs dict {(tile,k): sorted list of (in,out)})."""
    idx = [tuple(int(v) for v in r) for r in indices_sorted]
    oshape = list(shape) if subm else out_shape_of(shape, kernel, stride, padding)
    K0, K1, K2 = kernel
    cand = []
    for i, (b, x0, x1, x2) in enumerate(idx):
        for k0 in range(K0):
            for k1 in range(K1):
                for k2 in range(K2):
                    o = []
                    ok = True
                    for x, k, s, p, O in zip((x0, x1, x2), (k0, k1, k2), stride, padding, oshape):
                        t = x + p - k
                        if t % s != 0 or not (0 <= t // s < O):
                            ok = False
                            break
                        o.append(t // s)
                    if ok:
                        cand.append((i, (b, *o), (k0 * K1 + k1) * K2 + k2))
    if subm:
        out_coords = idx
    else:
        out_coords = sorted(set(c[1] for c in cand))
    row_of = {c: j for j, c in enumerate(out_coords)}
    tgw = -(-oshape[1] // tile[1])
    pairs = {}
    for i, oc, k in cand:
        j = row_of.get(oc)
        if j is None:
            continue
        t = (oc[1] // tile[0]) * tgw + (oc[2] // tile[1])
        pairs.setdefault((t, k), []).append((i, j))
    for v in pairs.values():
        v.sort()
    return np.array(out_coords, dtype=np.int32).reshape(-1, 4), pairs, oshape


def rules_to_dict(rules, rule_size):
    """Padded reference-format rules -> {(tile,k): sorted list of (in,out)}."""
    rules = np.asarray(rules)
    rule_size = np.asarray(rule_size)
    d = {}
    for t, k in zip(*np.nonzero(rule_size)):
        n = int(rule_size[t, k])
        d[(int(t), int(k))] = sorted(zip(rules[t, k, 0, :n].tolist(), rules[t, k, 1, :n].tolist()))
    return d


def dense_from_rows(feature, coords, B, shape, dtype=torch.float64):
    """[N,C] rows at coords [N,4] -> dense [B,C,S0,S1,S2]."""
    f = torch.as_tensor(np.asarray(feature), dtype=dtype)
    c = torch.as_tensor(np.asarray(coords), dtype=torch.long)
    dense = torch.zeros((B, f.shape[1], *shape), dtype=dtype)
    dense[c[:, 0], :, c[:, 1], c[:, 2], c[:, 3]] = f
    return dense


def dense_conv(dense_in, weight_kkkio, stride, padding, out_shape):
    """torch conv3d in float64; weight [K0,K1,K2,iC,oC] -> [oC,iC,K0,K1,K2]
    (the mapping the reference's test_grad.py:31 uses).  Cropped to out_shape
    (only matters for even kernels with padding K//2)."""
    w = torch.as_tensor(np.asarray(weight_kkkio), dtype=dense_in.dtype).permute(4, 3, 0, 1, 2)
    y = torch.nn.functional.conv3d(dense_in, w.contiguous(), None, tuple(stride), tuple(padding))
    return y[:, :, :out_shape[0], :out_shape[1], :out_shape[2]]


def gather_rows(dense, coords):
    c = torch.as_tensor(np.asarray(coords), dtype=torch.long)
    return dense[c[:, 0], :, c[:, 1], c[:, 2], c[:, 3]]
