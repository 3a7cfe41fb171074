"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

import helpers as H
from oracle import oracle as O
from sphconv_amd import _lib as L
from sphconv_amd.rulebook import RuleBook

DEV = "cuda:0"


def t(a, dtype=None):
    x = torch.as_tensor(np.ascontiguousarray(a)).to(DEV)
    return x if dtype is None else x.to(dtype)


def assert_same_conv(a, b):
    """Two convolution kernels on the same pairs (grouped and by-row form, one launch and two) may add a row's
    products in different orders: integer results are equal, floating-point results agree to the tolerance the
    path promises (fp32 rtol 1e-5; fp16/bf16 rtol 1e-2, atol 1e-3).  Run-to-run determinism of ONE kernel is
    asserted with torch.equal where it is tested."""
    a = a if torch.is_tensor(a) else torch.as_tensor(a)
    b = b if torch.is_tensor(b) else torch.as_tensor(b)
    assert a.shape == b.shape and a.dtype == b.dtype
    if not a.dtype.is_floating_point:
        assert torch.equal(a, b)
    elif a.dtype == torch.float32:
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5)   # atol: sums of products that cancel
    else:
        torch.testing.assert_close(a.float(), b.float(), rtol=1e-2, atol=1e-3)


def book_triples(buf):
    """Decode one book on the host -> int64 array [P,3] of (k, gather, owner),
    sorted by (k, owner).  Also checks the structural invariants of the layout."""
    torch.cuda.synchronize()
    nt, cap, kv = buf.ntiles, buf.cap, buf.kv
    if nt == 0:
        return np.zeros((0, 3), np.int64)
    ngrp = buf.tile_ngrp[:nt].cpu().numpy()
    koff = buf.tile_koff[:nt].cpu().numpy().astype(np.int64)
    gk = buf.grp_k.view(nt, cap).cpu().numpy()
    gat = buf.grp_gather.view(nt, cap, L.GROUP).cpu().numpy()
    own = buf.grp_owner.view(nt, cap, L.GROUP).cpu().numpy()
    assert (ngrp >= 0).all() and (ngrp <= cap).all()
    assert (koff[:, 0] == 0).all() and (koff[:, -1] == ngrp).all() and (np.diff(koff, axis=1) >= 0).all()
    used = np.arange(cap)[None, :] < ngrp[:, None]
    # grp_k agrees with tile_koff
    kk = np.repeat(np.arange(kv)[None, :], nt, 0)
    exp_k = np.full((nt, cap), -1, np.int64)
    for ti in range(nt):
        exp_k[ti, :ngrp[ti]] = np.repeat(kk[ti], np.diff(koff[ti]))
    assert (gk[used] == exp_k[used]).all()
    valid = used[:, :, None] & (own >= 0)
    assert ((gat >= 0) == (own >= 0))[used].all()
    # owner rows belong to their tile
    tile_of = np.arange(nt)[:, None, None]
    assert ((own // L.TILE_ROWS) == tile_of)[valid].all()
    # padding only at the tail of the last group of each k: within a (tile,k) list rows ascend
    k3 = np.broadcast_to(gk[:, :, None], own.shape)
    tri = np.stack([k3[valid], gat[valid], own[valid]], axis=1).astype(np.int64)
    order = np.lexsort((tri[:, 2], tri[:, 0]))
    # storage order inside the book is already (tile, k, owner) ascending
    flat_tile = np.broadcast_to(tile_of, own.shape)[valid]
    key = (flat_tile.astype(np.int64) * kv + tri[:, 0]) * (2 ** 31) + tri[:, 2]
    assert (np.diff(key) > 0).all()
    return tri[order]


def by_row_triples(buf):
    """The by-row form of a book -> [P,3] (k, gather, owner) sorted by (k, owner); None if not kept."""
    if buf.tile_nbr is None:
        return None
    torch.cuda.synchronize()
    nt, kv = buf.ntiles, buf.kv
    if nt == 0:
        return np.zeros((0, 3), np.int64)
    nbr = buf.tile_nbr[:nt].cpu().numpy()                      # [nt, kv, 128]
    t, k, r = np.nonzero(nbr >= 0)
    owner = t * L.TILE_ROWS + r
    assert (owner < buf.rows).all()
    tri = np.stack([k, nbr[t, k, r], owner], axis=1).astype(np.int64)
    return tri[np.lexsort((tri[:, 2], tri[:, 0]))]


def oracle_triples(rules, rule_size, swap=False):
    """Padded oracle rules -> [P,3] (k, in, out) sorted by (k, out)  (swap: (k, out, in) by (k, in))."""
    rules, rule_size = np.asarray(rules), np.asarray(rule_size)
    nt, kv, _, nmax = rules.shape
    m = np.arange(nmax)[None, None, :] < rule_size[:, :, None]
    k = np.broadcast_to(np.arange(kv)[None, :, None], m.shape)[m]
    i, o = rules[:, :, 0, :][m], rules[:, :, 1, :][m]
    tri = np.stack([k, o, i] if swap else [k, i, o], axis=1).astype(np.int64)
    order = np.lexsort((tri[:, 2], tri[:, 0]))
    return tri[order]


def build_case(idx, B, shape, kernel, stride, padding, subm):
    """COO indices -> (sorted indices, z_idx, z_ptr on host, device RuleBook, oracle outputs)."""
    sidx, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    if subm:
        padding = [k // 2 for k in kernel]
        stride = [1, 1, 1]
    oshape = list(shape) if subm else H.out_shape_of(shape, kernel, stride, padding)
    zi, zp = t(z_idx), t(z_ptr)
    if subm:
        book = RuleBook.build_subm(zi, zp, B, shape, kernel, padding)
    else:
        book = RuleBook.build(zi, zp, B, shape, oshape, kernel, stride, padding)
    fn = O.get_rules_subm if subm else O.get_rules
    ora = fn(z_idx, z_ptr, B, shape, oshape, kernel, stride, padding, (1, 1, 1), (2, 2))
    return dict(sidx=sidx, z_idx=z_idx, z_ptr=z_ptr, book=book, oracle=ora, oshape=oshape,
                padding=padding, stride=stride, kernel=kernel, B=B, shape=shape, subm=subm)
