"""GPU parity of the one-launch path (sph_rules_conv: rule generation + forward convolution of a layer) and of
the optional table of the rows' columns that the rule kernels take, all through the C ABI.

Rules are bit-exact against the oracle; convolution outputs are compared with the oracle's
(oracle/sphconv_oracle.c: orc_rule_conv_f32, following rule_conv_kernel.cu.h:91-153) at the tolerances of the
path: fp32 rtol 1e-5 (+ atol 1e-5 for sums that cancel), fp16/bf16 rtol 1e-2 / atol 1e-3 on rounded inputs,
int8 exact.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import gpu_helpers as G
import helpers as H
from oracle import oracle as O
from sphconv_amd import _lib as L
from sphconv_amd import sphconv_cuda as ext
from sphconv_amd.rulebook import RuleBook, _Buffers, row_columns
from sphconv_amd.synth import config2_with_voxels, make_config

pytestmark = pytest.mark.gpu


def _weights(rng, kv, ic, oc):
    return (rng.standard_normal((kv, ic, oc)) * np.sqrt(2.0 / (kv * ic))).astype(np.float32)


def _fused(case, feat_t, w_t, write_book, hint, scale=None):
    """sph_rules_conv on a case of gpu_helpers.build_case -> (out, buffers)."""
    lib = L.lib()
    book = case["book"]
    n, m = book.in_rows, book.out_rows
    kv, ic, oc = w_t.shape
    g = book.geom()
    buf = _Buffers(m, kv, G.DEV)
    for f in ("tile_ngrp", "grp_k", "grp_gather", "grp_owner"):
        getattr(buf, f).fill_(-7)
    packed = ext._packed_weight(w_t, False)
    out = torch.full((m, oc), 77, device=G.DEV).to(feat_t.dtype)
    epi = L.Epilogue(L.ptr(scale), None, 0)
    rc = lib.sph_rules_conv(L.ptr(book.z_idx), L.ptr(book.z_ptr), n, L.ptr(book.oz_idx), L.ptr(book.oz_ptr), m,
                            C.byref(g), C.byref(buf.struct()), int(write_book), L.ptr(hint), L.dtype_code(feat_t.dtype),
                            L.ptr(feat_t), ic, L.ptr(packed), oc, C.byref(epi), L.ptr(out), L.stream())
    L.check(rc)
    torch.cuda.synchronize()
    return out, buf


def _check_out(got, want, dtype):
    got = got.float().cpu().numpy()
    if dtype == torch.float32:
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    else:
        np.testing.assert_allclose(got, want, rtol=1e-2, atol=1e-3 * max(1.0, float(np.abs(want).max())))


def _random_indices(rng, B, shape, p):
    return np.argwhere(rng.random((B, *shape)) < p).astype(np.int32)


@pytest.mark.parametrize("subm,kernel,stride,padding,p,ic,oc,dtype", [
    (True, [3, 3, 3], [1, 1, 1], [1, 1, 1], 0.06, 16, 16, torch.float32),
    (True, [3, 3, 3], [1, 1, 1], [1, 1, 1], 0.04, 64, 64, torch.float16),
    (True, [3, 3, 3], [1, 1, 1], [1, 1, 1], 0.05, 32, 48, torch.bfloat16),
    (True, [3, 1, 3], [1, 1, 1], [1, 0, 1], 0.10, 8, 24, torch.float16),      # 16-byte rows: masked steps
    (False, [3, 3, 3], [2, 2, 2], [1, 1, 1], 0.08, 32, 64, torch.float16),
    (False, [2, 2, 2], [2, 2, 2], [0, 0, 0], 0.15, 16, 32, torch.float32),    # even kernel: no middle offset run
    (False, [3, 3, 3], [1, 2, 1], [1, 1, 1], 0.05, 32, 32, torch.float32),    # 128-byte fp32 rows into 32 columns
])
def test_one_launch_matches_the_oracle(subm, kernel, stride, padding, p, ic, oc, dtype):
    """Outputs against the oracle's convolution, the book it writes on request against the oracle's rules, with
    and without the table of the rows' columns."""
    rng = np.random.default_rng(ic * 7 + oc)
    B, shape = 3, [12, 40, 24]
    case = G.build_case(_random_indices(rng, B, shape, p), B, shape, kernel, stride, padding, subm)
    book = case["book"]
    n, m = book.in_rows, book.out_rows
    assert m > 3 * L.TILE_ROWS
    kv = kernel[0] * kernel[1] * kernel[2]
    feat = torch.tensor(rng.standard_normal((n, ic)), dtype=torch.float32).to(dtype)
    w = torch.tensor(_weights(rng, kv, ic, oc)).to(dtype)
    oz_idx, oz_ptr, rules, rule_size, dropped = case["oracle"]
    assert not dropped
    want = O.rule_conv(feat.float().numpy(), w.float().numpy(), rules, rule_size, m)
    cols = row_columns(book.oz_ptr, m)
    tri = G.oracle_triples(rules, rule_size)
    for hint in (None, cols):
        for flags in (0, L.FUSED_WRITE_BOOK, L.FUSED_IN_FLIGHT, L.FUSED_WRITE_BOOK | L.FUSED_IN_FLIGHT):
            out, buf = _fused(case, feat.to(G.DEV), w.to(G.DEV), flags, hint)
            _check_out(out, want, dtype)
            if flags & L.FUSED_WRITE_BOOK:
                assert np.array_equal(G.book_triples(buf), tri)
    # twice the same call: the same bits
    again, _ = _fused(case, feat.to(G.DEV), w.to(G.DEV), L.FUSED_WRITE_BOOK | L.FUSED_IN_FLIGHT, cols)
    assert torch.equal(again, out)


def test_one_launch_int8_exact():
    rng = np.random.default_rng(88)
    B, shape = 2, [16, 48, 16]
    case = G.build_case(_random_indices(rng, B, shape, 0.06), B, shape, [3, 3, 3], [1, 1, 1], [1, 1, 1], True)
    n = case["book"].in_rows
    f8 = rng.integers(-128, 128, (n, 64), dtype=np.int8)
    w8 = rng.integers(-128, 128, (27, 64, 64), dtype=np.int8)
    scale = ((rng.random(64) + 0.5) / 3000.0).astype(np.float32)
    _, _, rules, rule_size, _ = case["oracle"]
    want = O.rule_conv_i8(f8, w8, scale, rules, rule_size, n)
    out, _ = _fused(case, G.t(f8), G.t(w8), 0, None, scale=G.t(scale))
    assert np.array_equal(out.cpu().numpy(), want) and (np.abs(want) < 100).mean() > 0.3


def test_tiles_with_more_groups_than_the_workgroup_keeps_go_through_the_book():
    """A dense grid: 27 pairs per row, 216 groups per tile, far more than the kernel's LDS arrays hold; those
    tiles write their groups to the caller's book and convolve from there.  Same results."""
    rng = np.random.default_rng(5)
    B, shape = 1, [6, 20, 8]
    case = G.build_case(_random_indices(rng, B, shape, 1.1), B, shape, [3, 3, 3], [1, 1, 1], [1, 1, 1], True)
    n = case["book"].in_rows
    assert n == 6 * 20 * 8
    feat = torch.tensor(rng.standard_normal((n, 32)), dtype=torch.float32)
    w = torch.tensor(_weights(rng, 27, 32, 32))
    _, _, rules, rule_size, _ = case["oracle"]
    want = O.rule_conv(feat.numpy(), w.numpy(), rules, rule_size, n)
    for write_book in (0, 1):
        out, buf = _fused(case, feat.to(G.DEV), w.to(G.DEV), write_book, None)
        _check_out(out, want, torch.float32)
    assert np.array_equal(G.book_triples(buf), G.oracle_triples(rules, rule_size))


def test_shapes_the_one_launch_kernel_does_not_take_are_refused():
    rng = np.random.default_rng(6)
    B, shape = 1, [8, 16, 8]
    case = G.build_case(_random_indices(rng, B, shape, 0.2), B, shape, [3, 3, 3], [1, 1, 1], [1, 1, 1], True)
    n = case["book"].in_rows
    for ic, oc, dtype in ((12, 16, torch.float16), (128, 32, torch.float16), (32, 128, torch.float16), (64, 32, torch.float32)):
        feat = torch.zeros((n, ic), dtype=dtype, device=G.DEV)
        w = torch.zeros((27, ic, oc), dtype=dtype, device=G.DEV)
        with pytest.raises(L.SphconvError, match="status -2"):
            _fused(case, feat, w, 0, None)
        # the Python layer falls back to the two kernels by itself
        book = RuleBook.build_subm(case["book"].z_idx, case["book"].z_ptr, B, shape, [3, 3, 3], lazy=True)
        out = ext.rule_conv(feat, w, book, None, n)
        assert book.built and out.shape == (n, oc)


@pytest.mark.parametrize("subm,transposed", [(True, False), (False, False), (False, True)])
def test_a_wrong_table_of_columns_cannot_change_the_rules(subm, transposed):
    """sph_rules_build with the right table, no table, and tables that are shifted, random, out of range or
    partly wrong: the same book bit for bit (every entry is checked against z_ptr before it is believed)."""
    rng = np.random.default_rng(17 + subm + 2 * transposed)
    B, shape = 2, [16, 64, 12]
    kernel, stride, padding = [3, 3, 3], ([1, 1, 1] if subm else [2, 2, 2]), [1, 1, 1]
    case = G.build_case(_random_indices(rng, B, shape, 0.07), B, shape, kernel, stride, padding, subm)
    book = case["book"]
    lib = L.lib()
    g = book.geom()
    rows = book.in_rows if transposed else book.out_rows
    ptr = book.z_ptr if transposed else book.oz_ptr
    want = G.book_triples(book.transposed() if transposed else book.fwd)
    right = row_columns(ptr, rows)
    # the table itself: what numpy says
    counts = np.diff(np.concatenate([[0], ptr.cpu().numpy().reshape(-1)]))
    assert np.array_equal(right.cpu().numpy(), np.repeat(np.arange(counts.size), counts).astype(np.int32))
    partly = right.clone()
    partly[rng.integers(0, rows, 5)] += 1
    tables = [right, None, torch.roll(right, 1), partly, torch.full_like(right, -3), torch.full_like(right, 1 << 30),
              torch.tensor(rng.integers(0, ptr.numel(), rows), dtype=torch.int32, device=G.DEV)]
    for tab in tables:
        buf = _Buffers(rows, 27, G.DEV)
        L.check(lib.sph_rules_build(L.ptr(book.z_idx), L.ptr(book.z_ptr), book.in_rows, L.ptr(book.oz_idx), L.ptr(book.oz_ptr),
                                    book.out_rows, C.byref(g), int(transposed), C.byref(buf.struct()), L.ptr(tab), L.stream()))
        assert np.array_equal(G.book_triples(buf), want)


@pytest.mark.parametrize("which", ["config1", "headline", "120k"])
def test_one_launch_at_full_size(which):
    """The benchmark's own shapes through the one launch: 746 tiles (workgroups of four waves), 937 tiles (of two),
    configuration 1 in fp32, each against the oracle on the whole output."""
    if which == "config1":
        d, ic, oc, dtype = make_config(1, seed=0), 16, 16, torch.float32
    elif which == "headline":
        d, ic, oc, dtype = make_config(2, seed=0), 64, 64, torch.float16
    else:
        d, ic, oc, dtype = config2_with_voxels(120000, seed=0)[0], 64, 64, torch.float16
    shape, B = d["spatial_shape"], d["batch"]
    z_idx, z_ptr = d["z_idx"], d["z_ptr"]
    n = z_idx.shape[0]
    rng = np.random.default_rng(1)
    feat = torch.tensor(rng.standard_normal((n, ic)), dtype=torch.float32).to(dtype)
    w = torch.tensor(_weights(rng, 27, ic, oc)).to(dtype)
    zi, zp = G.t(z_idx), G.t(z_ptr)
    book = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3], row_cols=row_columns(zp, n), lazy=True)
    book.keep = False
    out = ext.rule_conv(feat.to(G.DEV), w.to(G.DEV), book, None, n)
    assert not book.built                   # one launch, no book
    _, _, rules, rule_size, dropped = O.get_rules_subm(z_idx, z_ptr, B, shape, shape, [3, 3, 3], [1, 1, 1], [1, 1, 1], n_max=256)
    assert not dropped
    want = O.rule_conv(feat.float().numpy(), w.float().numpy(), rules, rule_size, n)
    _check_out(out, want, dtype)
    # the book, when somebody asks for it afterwards, is generated then
    assert np.array_equal(G.book_triples(book.fwd), G.oracle_triples(rules, rule_size))
    assert book.built
