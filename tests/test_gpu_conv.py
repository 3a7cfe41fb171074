"""GPU parity of the convolution kernels (forward, dgrad, wgrad, int8) against
the CPU oracle, through the C ABI.

Tolerances (stated by the task): fp32 rtol 1e-5 (atol 1e-5 for sums that cancel);
fp16/bf16 storage with fp32 accumulate rtol 1e-2 / atol 1e-3 against a float64
evaluation on the rounded inputs, scaled by the row's absolute-sum magnitude
where outputs cancel; int8 bit-exact."""
import numpy as np
import pytest
import torch

import helpers as H
import gpu_helpers as G
from oracle import oracle as O
import sphconv_amd
from sphconv_amd import sphconv_cuda as ext
from sphconv_amd.synth import make_config

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("pair_form")]
CASES = H.load_ref_cases()


def _conv_calls():
    out = []
    for tc in CASES:
        if tc["file"] != "test/test_conv.py":
            continue
        for c in tc["calls"]:
            out.append(pytest.param(tc["tensors"][c["coords"]], c["args"],
                                    id="test_conv.py:%d" % c["line"]))
    return out


def _weights(rng, kv, ic, oc):
    return (rng.standard_normal((kv, ic, oc)) / np.sqrt(kv * ic)).astype(np.float32)


def _oracle_fwd(case, feat, w):
    oz_idx, _, rules, rule_size, _ = case["oracle"]
    return O.rule_conv(feat, w, rules, rule_size, oz_idx.shape[0])


@pytest.mark.parametrize("coords,args", _conv_calls())
def test_fp32_forward_reference_lists(coords, args):
    a = args
    subm = a.get("subm", False)
    idx = H.dup_with_batch_idx(coords, a["batch_size"])
    case = G.build_case(idx, a["batch_size"], a["spatial_shape_DWH"], a["kernel_size"], a["stride"],
                        a["padding"], subm)
    rng = np.random.default_rng(1)
    ic, oc, kv = a["in_channels"], a["out_channels"], int(np.prod(a["kernel_size"]))
    feat = rng.standard_normal((case["sidx"].shape[0], ic)).astype(np.float32)
    w = _weights(rng, kv, ic, oc)
    book = case["book"]
    out = ext.rule_conv(G.t(feat), G.t(w), book, None, book.out_rows).cpu().numpy()
    np.testing.assert_allclose(out, _oracle_fwd(case, feat, w), rtol=1e-5, atol=1e-5)
    # the reference-format entry: padded rules + rule_size through the same call
    rules, rule_size = book.padded((2, 2))
    out2 = ext.rule_conv(G.t(feat), G.t(w), rules, rule_size, book.out_rows).cpu().numpy()
    G.assert_same_conv(out, out2)      # by groups here, by rows above when that form is forced
    # and against torch's dense conv3d in float64
    dense = H.dense_from_rows(feat, case["sidx"], case["B"], case["shape"])
    y = H.dense_conv(dense, w.reshape(*a["kernel_size"], ic, oc), case["stride"], case["padding"], case["oshape"])
    out_coords, _, _ = H.brute_rules(case["sidx"], case["B"], case["shape"], a["kernel_size"],
                                     case["stride"], case["padding"], subm)
    np.testing.assert_allclose(out, H.gather_rows(y, out_coords).numpy(), rtol=1e-4, atol=1e-5)


def _random_case(seed, subm, kernel=(3, 3, 3), stride=(2, 2, 2), padding=(1, 1, 1), B=2,
                 shape=(11, 40, 24), p=0.25):
    rng = np.random.default_rng(seed)
    occ = rng.random((B, *shape)) < p
    idx = np.argwhere(occ).astype(np.int32)
    return G.build_case(idx, B, list(shape), list(kernel), list(stride), list(padding), subm)


CHANNELS = [(1, 1), (3, 5), (4, 4), (5, 8), (16, 16), (17, 33), (32, 32), (32, 64), (64, 64), (64, 128),
            (128, 64), (100, 20)]


@pytest.mark.parametrize("ic,oc", CHANNELS)
@pytest.mark.parametrize("subm", [True, False])
def test_fp32_forward_channels(ic, oc, subm):
    case = _random_case(ic * 131 + oc, subm)
    rng = np.random.default_rng(2)
    feat = rng.standard_normal((case["sidx"].shape[0], ic)).astype(np.float32)
    w = _weights(rng, 27, ic, oc)
    book = case["book"]
    out = ext.rule_conv(G.t(feat), G.t(w), book, None, book.out_rows).cpu().numpy()
    np.testing.assert_allclose(out, _oracle_fwd(case, feat, w), rtol=1e-5, atol=1e-5)


def _f64_pair_sum(case, feat64, w64, transposed=False):
    """sum over oracle pairs in float64 (definition), vectorised per (k)."""
    oz_idx, _, rules, rule_size, _ = case["oracle"]
    tri = G.oracle_triples(rules, rule_size)
    if not transposed:
        out = np.zeros((oz_idx.shape[0], w64.shape[2]))
        absacc = np.zeros_like(out)
        for k in np.unique(tri[:, 0]):
            s = tri[tri[:, 0] == k]
            out[s[:, 2]] += feat64[s[:, 1]] @ w64[k]
            absacc[s[:, 2]] += np.abs(feat64[s[:, 1]]) @ np.abs(w64[k])
    else:
        out = np.zeros((case["sidx"].shape[0], w64.shape[1]))
        absacc = np.zeros_like(out)
        for k in np.unique(tri[:, 0]):
            s = tri[tri[:, 0] == k]
            out[s[:, 1]] += feat64[s[:, 2]] @ w64[k].T
            absacc[s[:, 1]] += np.abs(feat64[s[:, 2]]) @ np.abs(w64[k]).T
    return out, absacc


@pytest.mark.parametrize("subm,p", [(True, 0.25), (True, 0.012), (True, 0.9), (False, 0.25)])
@pytest.mark.parametrize("dtype,ic,oc", [(torch.float32, 16, 16), (torch.float16, 64, 64), (torch.bfloat16, 32, 48),
                                         (torch.float16, 8, 64), (torch.int8, 64, 64)])
def test_middle_run_is_a_hint_not_a_contract(subm, p, dtype, ic, oc):
    """sph_conv_apply with and without sph_book.middle_run (helper waves for the middle offset's groups) against the
    oracle: submanifold books with full runs, with tiles whose middle offset holds one group or none (the helper
    waves leave), nearly full grids (tiles of more than 64 groups), and a strided book, which has no run whatever the
    caller claims.  Integers equal, floating point to the path's tolerance; each setting twice, bit for bit."""
    import ctypes as C
    from sphconv_amd import _lib as L
    case = _random_case(int(p * 1000) + ic + 7 * oc, subm, p=p, shape=(9, 36, 20))
    book = case["book"]
    n, m = book.in_rows, book.out_rows
    rng = np.random.default_rng(5)
    if dtype == torch.int8:
        feat = torch.tensor(rng.integers(-128, 128, (n, ic)), dtype=torch.int8)
        w = torch.tensor(rng.integers(-128, 128, (27, ic, oc)), dtype=torch.int8)
        scale = torch.tensor((rng.random(oc) + 0.5) / 3000.0, dtype=torch.float32)
        want = O.rule_conv_i8(feat.numpy(), w.numpy(), scale.numpy(), case["oracle"][2], case["oracle"][3], m)
    else:
        feat = torch.tensor(rng.standard_normal((n, ic)), dtype=torch.float32).to(dtype)
        w = torch.tensor(_weights(rng, 27, ic, oc)).to(dtype)
        scale = None
        want = _oracle_fwd(case, feat.float().numpy(), w.float().numpy())
    feat, w = feat.to(G.DEV), w.to(G.DEV)
    packed = ext._packed_weight(w, False)
    sc_keep = scale.to(G.DEV) if scale is not None else None
    epi = L.Epilogue(L.ptr(sc_keep), None, 0)
    bk = book.fwd.struct()
    outs = []
    for flag in (0, 1, 0, 1):
        bk.middle_run = flag
        out = torch.full((m, oc), 3, device=G.DEV).to(dtype)
        L.check(L.lib().sph_conv_apply(L.dtype_code(dtype), L.ptr(feat), n, ic, L.ptr(packed), oc, C.byref(bk), C.byref(epi),
                                       L.ptr(out), L.stream()))
        torch.cuda.synchronize()
        outs.append(out)
    bk.middle_run = int(subm)
    assert torch.equal(outs[0], outs[2]) and torch.equal(outs[1], outs[3])
    G.assert_same_conv(outs[0], outs[1])
    for out in outs[:2]:
        if dtype == torch.int8:
            assert np.array_equal(out.cpu().numpy(), want)
        elif dtype == torch.float32:
            np.testing.assert_allclose(out.cpu().numpy(), want, rtol=1e-5, atol=1e-5)
        else:
            np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-3 * max(1.0, float(np.abs(want).max())))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ic,oc", [(4, 4), (16, 16), (32, 32), (32, 64), (64, 64), (24, 40), (128, 128)])
@pytest.mark.parametrize("subm", [True, False])
def test_half_forward(dtype, ic, oc, subm):
    case = _random_case(7 + ic + oc, subm)
    rng = np.random.default_rng(3)
    feat = torch.tensor(rng.standard_normal((case["sidx"].shape[0], ic)), dtype=torch.float32).to(dtype)
    w = torch.tensor(_weights(rng, 27, ic, oc)).to(dtype)
    book = case["book"]
    out = ext.rule_conv(feat.to(G.DEV), w.to(G.DEV), book, None, book.out_rows)
    assert out.dtype == dtype
    ref, mag = _f64_pair_sum(case, feat.double().numpy(), w.double().numpy())
    # output rounding: half an ulp of the storage type relative to the value
    eps = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    err = np.abs(out.double().cpu().numpy() - ref)
    assert (err <= 1e-3 + 1e-2 * np.abs(ref)).all()
    assert (err <= 1e-6 + 2 * eps * np.abs(ref) + 1e-5 * mag).all()     # fp32 accumulate, one rounding


@pytest.mark.parametrize("ic,oc", [(16, 8), (64, 64), (20, 36), (128, 128)])
@pytest.mark.parametrize("subm", [True, False])
def test_int8_forward_exact(ic, oc, subm):
    case = _random_case(11 + ic, subm)
    rng = np.random.default_rng(4)
    n = case["sidx"].shape[0]
    f8 = rng.integers(-128, 128, (n, ic), dtype=np.int8)
    w8 = rng.integers(-128, 128, (27, ic, oc), dtype=np.int8)
    scale = ((rng.random(oc) + 0.5) / (40.0 * ic)).astype(np.float32)
    oz_idx, _, rules, rule_size, _ = case["oracle"]
    want = O.rule_conv_i8(f8, w8, scale, rules, rule_size, oz_idx.shape[0])
    book = case["book"]
    got = ext.rule_conv_int8(G.t(f8), G.t(w8), G.t(scale), book, None, book.out_rows).cpu().numpy()
    assert got.dtype == np.int8
    assert np.array_equal(got, want)
    assert want.min() == -128 and want.max() == 127 and (np.abs(want) < 100).mean() > 0.3


def test_int8_more_than_64_columns_on_more_than_1024_tiles():
    """int8 64 -> 128 on more than 131 072 rows: the grouped kernel's two-waves-per-tile form is for up to 64
    output columns only (more would be four waves per tile, beyond its launch bound); bit-exact."""
    rng = np.random.default_rng(64128)
    B, shape = 8, [32, 128, 32]
    idx = np.argwhere(rng.random((B, *shape)) < 0.14).astype(np.int32)
    case = G.build_case(idx, B, shape, [3, 3, 3], [1, 1, 1], [1, 1, 1], True)
    n = case["sidx"].shape[0]
    assert n > 1024 * 128
    f8 = rng.integers(-128, 128, (n, 64), dtype=np.int8)
    w8 = rng.integers(-128, 128, (27, 64, 128), dtype=np.int8)
    scale = ((rng.random(128) + 0.5) / 3000.0).astype(np.float32)
    _, _, rules, rule_size, dropped = O.get_rules_subm(case["z_idx"], case["z_ptr"], B, shape, shape, [3, 3, 3],
                                                       [1, 1, 1], [1, 1, 1], n_max=512)
    assert dropped == 0
    want = O.rule_conv_i8(f8, w8, scale, rules, rule_size, n)
    got = ext.rule_conv_int8(G.t(f8), G.t(w8), G.t(scale), case["book"], None, n).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("ic,oc", [(4, 4), (16, 16), (32, 64), (64, 64), (9, 21)])
@pytest.mark.parametrize("subm,kernel,stride,padding", [
    (True, (3, 3, 3), (1, 1, 1), (1, 1, 1)),
    (False, (3, 3, 3), (2, 2, 2), (1, 1, 1)),
    (False, (2, 2, 1), (1, 1, 1), (0, 0, 0)),
    (True, (1, 1, 1), (1, 1, 1), (0, 0, 0)),      # one offset: the centre is the only one
    (True, (5, 5, 5), (1, 1, 1), (2, 2, 2)),      # kernel volume 125
])
def test_fp32_backward(ic, oc, subm, kernel, stride, padding):
    case = _random_case(21 + ic, subm, kernel, stride, padding)
    rng = np.random.default_rng(5)
    kv = int(np.prod(kernel))
    n, m = case["sidx"].shape[0], case["oracle"][0].shape[0]
    feat = rng.standard_normal((n, ic)).astype(np.float32)
    w = _weights(rng, kv, ic, oc)
    g = rng.standard_normal((m, oc)).astype(np.float32)
    w_perm = np.ascontiguousarray(w.transpose(0, 2, 1))
    _, _, rules, rule_size, _ = case["oracle"]
    tgs = [-(-case["oshape"][0] // 2), -(-case["oshape"][1] // 2)]
    d_feat_o, d_w_o = O.rule_conv_backward(g, feat, w_perm, rules, rule_size, tgs)
    book = case["book"]
    # reference entry point: weight pre-permuted to [KV,oC,iC]
    d_feat, d_w = ext.rule_conv_backward(G.t(g), G.t(feat), G.t(w_perm), book, None, tgs)
    # a submanifold book with odd kernels is its own transpose (offsets mirrored): no second book is built
    assert (book._bwd is None) == book.mirrored() and book.mirrored() == (subm and all(k % 2 for k in kernel))
    np.testing.assert_allclose(d_feat.cpu().numpy(), d_feat_o, rtol=1e-5, atol=1e-5)
    # d_weight sums thousands of products that cancel: both fp32 evaluations (oracle and
    # GPU, different association) are held to 1e-5 of the sum of absolute products,
    # measured against the float64 definition
    tri = G.oracle_triples(rules, rule_size)
    dw64 = np.zeros((kv, ic, oc))
    mag = np.zeros((kv, ic, oc))
    f64, g64 = feat.astype(np.float64), g.astype(np.float64)
    for k in np.unique(tri[:, 0]):
        s = tri[tri[:, 0] == k]
        dw64[k] = f64[s[:, 1]].T @ g64[s[:, 2]]
        mag[k] = np.abs(f64[s[:, 1]]).T @ np.abs(g64[s[:, 2]])
    assert (np.abs(d_w.cpu().numpy() - dw64) <= 1e-5 * mag + 1e-6).all()
    assert (np.abs(d_w_o - dw64) <= 1e-5 * mag + 1e-6).all()
    # same through padded rules
    pr, ps = book.padded((2, 2))
    d_feat2, d_w2 = ext.rule_conv_backward(G.t(g), G.t(feat), G.t(w_perm), pr, ps, tgs)
    if book.mirrored():   # dgrad ran on the forward book with mirrored offsets: same pairs, another order of summation
        np.testing.assert_allclose(d_feat2.cpu().numpy(), d_feat.cpu().numpy(), rtol=1e-5, atol=1e-5)
    else:
        G.assert_same_conv(d_feat2, d_feat)
    assert np.array_equal(d_w2.cpu().numpy(), d_w.cpu().numpy())
    # float64 definition
    ref, _ = _f64_pair_sum(case, g.astype(np.float64), w.astype(np.float64), transposed=True)
    np.testing.assert_allclose(d_feat.cpu().numpy(), ref, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_half_backward(dtype):
    case = _random_case(31, True, p=0.3)
    rng = np.random.default_rng(6)
    n = case["sidx"].shape[0]
    feat = torch.tensor(rng.standard_normal((n, 64)), dtype=torch.float32).to(dtype)
    w = torch.tensor(_weights(rng, 27, 64, 64)).to(dtype)
    g = torch.tensor(rng.standard_normal((n, 64)), dtype=torch.float32).to(dtype)
    book = case["book"]
    d_feat, d_w = ext.rule_conv_backward(g.to(G.DEV), feat.to(G.DEV),
                                         w.permute(0, 2, 1).contiguous().to(G.DEV), book, None, [1, 1])
    ref, _ = _f64_pair_sum(case, g.double().numpy(), w.double().numpy(), transposed=True)
    err = np.abs(d_feat.double().cpu().numpy() - ref)
    assert (err <= 1e-3 + 1e-2 * np.abs(ref)).all()
    tri = G.oracle_triples(case["oracle"][2], case["oracle"][3])
    dw_ref = np.zeros((27, 64, 64))
    f64, g64 = feat.double().numpy(), g.double().numpy()
    for k in range(27):
        s = tri[tri[:, 0] == k]
        dw_ref[k] = f64[s[:, 1]].T @ g64[s[:, 2]]
    err = np.abs(d_w.double().cpu().numpy() - dw_ref)
    assert (err <= 1e-3 + 1e-2 * np.abs(dw_ref) + 2e-3 * np.sqrt(n)).all()


@pytest.mark.parametrize("dtype,ic,oc", [
    (torch.float16, 8, 24), (torch.float16, 40, 64), (torch.float16, 16, 32),
    (torch.bfloat16, 128, 64), (torch.bfloat16, 64, 128), (torch.bfloat16, 96, 48),
    (torch.float32, 72, 40), (torch.float32, 128, 128), (torch.float32, 4, 12),
    (torch.float16, 6, 10), (torch.bfloat16, 3, 17),      # rows that are no whole 16-byte chunks: the general kernel
])
@pytest.mark.parametrize("subm", [True, False])
def test_wgrad_channel_blocks_and_chunks(dtype, ic, oc, subm):
    """Weight gradient over more than 64 tiles (several chunks, more than four slices at
    the centre offset) and over channel counts that need several 64x64 blocks, zero-padded
    16-channel tiles, or the general kernel (rows that are not whole 16-byte chunks)."""
    case = _random_case(500 + ic + oc, subm, shape=(16, 64, 24), p=0.3)
    rng = np.random.default_rng(8)
    n, m = case["sidx"].shape[0], case["oracle"][0].shape[0]
    assert max(n, m) > 64 * 128
    feat = torch.tensor(rng.standard_normal((n, ic)), dtype=torch.float32).to(dtype)
    g = torch.tensor(rng.standard_normal((m, oc)), dtype=torch.float32).to(dtype)
    book = case["book"]
    d_w = ext.rule_conv_d_weight(feat.to(G.DEV), g.to(G.DEV), book, None)
    assert d_w.dtype == dtype and tuple(d_w.shape) == (27, ic, oc)
    tri = G.oracle_triples(case["oracle"][2], case["oracle"][3])
    f64, g64 = feat.double().numpy(), g.double().numpy()
    ref = np.zeros((27, ic, oc))
    mag = np.zeros((27, ic, oc))
    for k in np.unique(tri[:, 0]):
        s = tri[tri[:, 0] == k]
        ref[k] = f64[s[:, 1]].T @ g64[s[:, 2]]
        mag[k] = np.abs(f64[s[:, 1]]).T @ np.abs(g64[s[:, 2]])
    err = np.abs(d_w.double().cpu().numpy() - ref)
    # fp32 accumulation of the products (1e-5 of their absolute sum) + one rounding to the storage type
    eps = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    assert (err <= 1e-5 * mag + 2 * eps * np.abs(ref) + 1e-6).all()
    # run-to-run determinism (fixed summation order)
    again = ext.rule_conv_d_weight(feat.to(G.DEV), g.to(G.DEV), book, None)
    assert torch.equal(again, d_w)
    # the same reduction stored as fp32 (an fp32 master weight): no rounding to the storage type, and rounding
    # it afterwards gives the typed result bit for bit
    wide = ext.rule_conv_d_weight(feat.to(G.DEV), g.to(G.DEV), book, None, torch.float32)
    assert wide.dtype == torch.float32
    assert torch.equal(wide.to(dtype), d_w)
    assert (np.abs(wide.double().cpu().numpy() - ref) <= 1e-5 * mag + 1e-6).all()


@pytest.mark.parametrize("dtype,ic,oc,subm", [(torch.float32, 16, 32, True), (torch.float16, 32, 64, True),
                                              (torch.bfloat16, 64, 64, False), (torch.float16, 20, 24, False),
                                              (torch.float32, 5, 7, True)])
def test_fused_epilogue_scale_shift_relu(dtype, ic, oc, subm):
    """y = relu(acc * scale[c] + shift[c]) in the convolution's store, against the ORACLE's accumulator with the
    affine and the ReLU applied in float64 (fast and general kernels, submanifold and strided books, with either
    of scale / shift missing and without ReLU), and against the unfused device result."""
    case = _random_case(41 + ic, subm)
    rng = np.random.default_rng(7)
    n, m = case["sidx"].shape[0], case["book"].out_rows
    feat = torch.tensor(rng.standard_normal((n, ic)).astype(np.float32)).to(dtype)
    w = torch.tensor(_weights(rng, 27, ic, oc)).to(dtype)
    scale = (rng.random(oc) + 0.5).astype(np.float32)
    shift = rng.standard_normal(oc).astype(np.float32)
    book = case["book"]
    acc = _oracle_fwd(case, feat.float().numpy(), w.float().numpy()).astype(np.float64)   # on the rounded inputs
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-3 * max(1.0, np.abs(acc).max()))
    fd, wd = feat.to(G.DEV), w.to(G.DEV)
    for use_scale, use_shift, relu in ((True, True, True), (True, False, False), (False, True, True), (True, True, False)):
        want = acc * (scale if use_scale else 1.0) + (shift if use_shift else 0.0)
        if relu:
            want = np.maximum(want, 0.0)
        got = ext.rule_conv(fd, wd, book, None, m, scale=G.t(scale) if use_scale else None,
                            shift=G.t(shift) if use_shift else None, relu=relu)
        assert got.dtype == dtype
        np.testing.assert_allclose(got.double().cpu().numpy(), want, **tol)
    if dtype == torch.float32:
        plain = ext.rule_conv(fd, wd, book, None, m)
        fused = ext.rule_conv(fd, wd, book, None, m, scale=G.t(scale), shift=G.t(shift), relu=True)
        torch.testing.assert_close(fused, torch.relu(plain * G.t(scale) + G.t(shift)), rtol=1e-6, atol=1e-6)


def test_stable_case_extreme_weights():
    """Reference test_stable.py:15-194: 74 voxels, stride 2, 64->64, extreme weights."""
    tc = [c for c in CASES if c["file"] == "test/test_stable.py"][0]
    coords = np.array(tc["tensors"]["indices_bzyx"], np.int32)
    case = G.build_case(coords, 1, [6, 6, 20], [3, 3, 3], [2, 2, 2], [1, 1, 1], False)
    raw = np.full((coords.shape[0], 64), 100.0, np.float32)
    raw[0, :] = 8.0
    raw[3, :] = 16.0
    _, order = H.canonical_rows(coords)
    feat = raw[order]
    w = (np.random.default_rng(0).standard_normal((3, 3, 3, 64, 64)) / 2).astype(np.float32)
    w[1] = 8.0
    w[-1] = 100.0
    w[1, 2, 0, :5, :] = 1 / 64
    book = case["book"]
    out = ext.rule_conv(G.t(feat), G.t(w.reshape(27, 64, 64)), book, None, book.out_rows).cpu().numpy()
    want = _oracle_fwd(case, feat, w.reshape(27, 64, 64))
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-2)
    # run-to-run determinism (reference test_stable.py repeats the call)
    for _ in range(3):
        again = ext.rule_conv(G.t(feat), G.t(w.reshape(27, 64, 64)), book, None, book.out_rows).cpu().numpy()
        assert np.array_equal(again, out)


def test_config1_full_size_fp32():
    """BASELINE config 1 at full size against the oracle (C, fp32)."""
    d = make_config(1, seed=0)
    shape, B = d["spatial_shape"], d["batch"]
    rng = np.random.default_rng(0)
    n = d["z_idx"].shape[0]
    feat = rng.standard_normal((n, 16)).astype(np.float32)
    w = _weights(rng, 27, 16, 16)
    from sphconv_amd.rulebook import RuleBook
    book = RuleBook.build_subm(G.t(d["z_idx"]), G.t(d["z_ptr"]), B, shape, [3, 3, 3])
    out = ext.rule_conv(G.t(feat), G.t(w), book, None, n).cpu().numpy()
    _, _, rules, rule_size, dropped = O.get_rules_subm(d["z_idx"], d["z_ptr"], B, shape, shape, [3, 3, 3],
                                                       [1, 1, 1], [1, 1, 1], n_max=256)
    assert dropped == 0
    want = O.rule_conv(feat, w, rules, rule_size, n)
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-5)


def _full_size_case(cfg):
    from sphconv_amd.rulebook import RuleBook
    d = make_config(cfg, seed=0)
    shape, B = d["spatial_shape"], d["batch"]
    subm = cfg != 3
    zi, zp = G.t(d["z_idx"]), G.t(d["z_ptr"])
    if subm:
        oshape = shape
        book = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3])
        ora = O.get_rules_subm(d["z_idx"], d["z_ptr"], B, shape, shape, [3, 3, 3], [1, 1, 1], [1, 1, 1], n_max=512)
    else:
        oshape = H.out_shape_of(shape, [3, 3, 3], [2, 2, 2], [1, 1, 1])
        book = RuleBook.build(zi, zp, B, shape, oshape, [3, 3, 3], [2, 2, 2], [1, 1, 1])
        ora = O.get_rules(d["z_idx"], d["z_ptr"], B, shape, oshape, [3, 3, 3], [2, 2, 2], [1, 1, 1], n_max=512)
    assert ora[4] == 0                                   # no pair dropped by the oracle's padded lists
    return d, book, ora


@pytest.mark.parametrize("cfg,ic,oc,dtype,backward", [
    (2, 32, 32, torch.float16, False), (3, 32, 64, torch.float16, True), (5, 64, 64, torch.float16, True),
    (2, 64, 64, torch.float16, True),      # the shape the benchmark times: configuration 2's grid at 64 -> 64
    (2, 64, 64, torch.bfloat16, True), (3, 32, 64, torch.bfloat16, False)],
    ids=["cfg2-32-32-f16", "cfg3-32-64-f16", "cfg5b-64-64-f16", "headline-64-64-f16", "headline-64-64-bf16",
         "cfg3-32-64-bf16"])
def test_configs_full_size_fp16(cfg, ic, oc, dtype, backward):
    """BASELINE configurations 2, 3, 5b and the benchmark's shape (configuration 2's grid, 64 -> 64) at full
    size: fp16 / bf16 storage with fp32 accumulate against the C oracle (fp32) on the same rounded inputs;
    3 (fp16), 5b and the benchmark's shape also dgrad and wgrad."""
    d, book, (oz_idx, _, rules, rule_size, _) = _full_size_case(cfg)
    rng = np.random.default_rng(cfg)
    n, m = d["z_idx"].shape[0], oz_idx.shape[0]
    ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7   # one rounding to the storage type
    feat = torch.tensor(rng.standard_normal((n, ic)), dtype=torch.float32).to(dtype)
    w = torch.tensor(_weights(rng, 27, ic, oc)).to(dtype)
    out = ext.rule_conv(feat.to(G.DEV), w.to(G.DEV), book, None, m)
    assert out.dtype == dtype and tuple(out.shape) == (m, oc)
    want = O.rule_conv(feat.float().numpy(), w.float().numpy(), rules, rule_size, m)
    got = out.float().cpu().numpy()
    # one rounding of an fp32 sum of at most 27*ic products (tolerance of north_star: 1e-2 relative)
    assert (np.abs(got - want) <= ulp * np.abs(want) + 1e-3).all()
    if not backward:
        return
    g = torch.tensor(rng.standard_normal((m, oc)), dtype=torch.float32).to(dtype)
    w_perm = w.permute(0, 2, 1).contiguous()
    d_feat, d_w = ext.rule_conv_backward(g.to(G.DEV), feat.to(G.DEV), w_perm.to(G.DEV), book, None, [1, 1])
    tgs = [-(-book.out_shape[0] // 2), -(-book.out_shape[1] // 2)]    # tiles of 2 x 2 output columns
    df_o, dw_o = O.rule_conv_backward(g.float().numpy(), feat.float().numpy(), w_perm.float().numpy(), rules,
                                      rule_size, tgs)
    assert (np.abs(d_feat.float().cpu().numpy() - df_o) <= ulp * np.abs(df_o) + 1e-3).all()
    # d_weight sums ~23 000 products per entry (centre offset: 314 000).  Held against the float64 sum over the
    # oracle's pairs: the fp32 accumulation may be off by 1e-5 of the sum of the products' magnitudes (computed,
    # not estimated), the stored value by one more rounding to the storage type.  A partial sum that had gone
    # through 16 bits on the way (error ~ ulp x magnitude of the partial sums) does not fit that bound.
    tri = torch.tensor(G.oracle_triples(rules, rule_size), device=G.DEV)
    f64, g64 = feat.to(G.DEV).double(), g.to(G.DEV).double()
    dw64 = torch.zeros((27, ic, oc), dtype=torch.float64, device=G.DEV)
    mag = torch.zeros_like(dw64)
    for k in range(27):
        sel = tri[tri[:, 0] == k]
        fi, go = f64[sel[:, 1]], g64[sel[:, 2]]
        dw64[k] = fi.T @ go
        mag[k] = fi.abs().T @ go.abs()
    dw64, mag = dw64.cpu().numpy(), mag.cpu().numpy()
    assert (np.abs(d_w.float().cpu().numpy() - dw64) <= 1e-5 * mag + ulp * np.abs(dw64) + 1e-6).all()
    assert (np.abs(dw_o - dw64) <= 1e-5 * mag + 1e-6).all()
    # the fp32 form of the same gradient (an fp32 master weight): no rounding to the storage type at all
    d_w32 = ext.rule_conv_d_weight(feat.to(G.DEV), g.to(G.DEV), book, None, torch.float32)
    assert d_w32.dtype == torch.float32
    assert (np.abs(d_w32.cpu().numpy() - dw64) <= 1e-5 * mag + 1e-6).all()


def test_config5a_full_size_int8_exact():
    """BASELINE configuration 5a at full size: int8 x int8 -> int32 -> requantised int8, bit-exact."""
    d, book, (oz_idx, _, rules, rule_size, _) = _full_size_case(5)
    rng = np.random.default_rng(55)
    n = d["z_idx"].shape[0]
    f8 = rng.integers(-128, 128, (n, 64), dtype=np.int8)
    w8 = rng.integers(-128, 128, (27, 64, 64), dtype=np.int8)
    scale = ((rng.random(64) + 0.5) / 3000.0).astype(np.float32)
    want = O.rule_conv_i8(f8, w8, scale, rules, rule_size, n)
    got = ext.rule_conv_int8(G.t(f8), G.t(w8), G.t(scale), book, None, n).cpu().numpy()
    assert np.array_equal(got, want)
    assert (want == 127).any() and (want == -128).any() and (np.abs(want) < 100).mean() > 0.3


def test_errors_are_reported_not_fatal():
    from sphconv_amd import SphconvError
    case = _random_case(51, True)
    n = case["sidx"].shape[0]
    book = case["book"]
    with pytest.raises(SphconvError):
        ext.rule_conv(torch.zeros((n, 8), device=G.DEV), torch.zeros((27, 8, 200), device=G.DEV), book, None, n)
    with pytest.raises(SphconvError):
        ext.rule_conv(torch.zeros((n, 8), device=G.DEV), torch.zeros((27, 9, 8), device=G.DEV), book, None, n)
    with pytest.raises(SphconvError):
        ext.rule_conv(torch.zeros((n, 8), device=G.DEV, dtype=torch.float64),
                      torch.zeros((27, 8, 8), device=G.DEV, dtype=torch.float64), book, None, n)
    with pytest.raises(SphconvError):
        ext.rule_conv(torch.zeros((n, 8)), torch.zeros((27, 8, 8)), book, None, n)   # CPU tensors


@pytest.mark.parametrize("dtype,ic,oc", [(torch.float16, 64, 64), (torch.float32, 5, 33), (torch.int8, 32, 16),
                                         (torch.bfloat16, 128, 96)])
@pytest.mark.parametrize("subm", [True, False])
def test_weight_packed_by_the_rule_launch(dtype, ic, oc, subm):
    """The weight copy made by extra workgroups of the rule kernel launch equals sph_weight_pack's,
    the book equals the one built alone, and rule_conv(packed=) gives the same output bits."""
    from sphconv_amd.rulebook import RuleBook
    case = _random_case(900 + ic, subm)
    rng = np.random.default_rng(9)
    if dtype == torch.int8:
        w = torch.tensor(rng.integers(-128, 128, (27, ic, oc)), dtype=torch.int8)
    else:
        w = torch.tensor(_weights(rng, 27, ic, oc)).to(dtype)
    w = w.to(G.DEV)
    zi, zp = G.t(case["z_idx"]), G.t(case["z_ptr"])
    if subm:
        book, packed = RuleBook.build_subm(zi, zp, case["B"], case["shape"], case["kernel"], weight=w)
    else:
        book, packed = RuleBook.build(zi, zp, case["B"], case["shape"], case["oshape"], case["kernel"],
                                      case["stride"], case["padding"], weight=w)
    assert torch.equal(packed, ext._packed_weight(w, False))
    assert np.array_equal(G.book_triples(book.fwd), G.book_triples(case["book"].fwd))
    if dtype == torch.int8:
        return
    feat = torch.tensor(rng.standard_normal((zi.shape[0], ic)), dtype=torch.float32).to(dtype).to(G.DEV)
    a = ext.rule_conv(feat, w, book, None, book.out_rows, packed=packed)
    b = ext.rule_conv(feat, w, case["book"], None, book.out_rows)
    assert torch.equal(a, b)
    with pytest.raises(sphconv_amd.SphconvError):
        ext.rule_conv(feat, w, book, None, book.out_rows, packed=packed[:-1024])


def test_forward_only_book_builds_its_groups_on_demand(pair_form):
    """A by-row book made for a forward pass without gradients leaves its groups out; wgrad, the padded
    tensors and a call that cannot go by rows build them when they are asked for."""
    from sphconv_amd.rulebook import RuleBook
    rng = np.random.default_rng(21)
    B, shape = 2, [6, 10, 8]
    occ = rng.random((B, *shape)) < 0.5
    idx = np.argwhere(occ).astype(np.int32)
    _, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    n = z_idx.shape[0]
    feat = torch.tensor(rng.standard_normal((n, 32)), dtype=torch.float32).half().to(G.DEV)
    w = torch.tensor(_weights(rng, 27, 32, 16)).half().to(G.DEV)
    zi, zp = G.t(z_idx), G.t(z_ptr)
    ref_book = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3])
    want = ext.rule_conv(feat, w, ref_book, None, n)
    with torch.no_grad():
        book, packed = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3], weight=w)
    assert book.fwd.groups == (pair_form == "groups")
    assert book.num_pairs() == ref_book.num_pairs()
    got = ext.rule_conv(feat, w, book, None, n, packed=packed)
    G.assert_same_conv(got, want)
    # 12 fp16 input channels are 24-byte rows: not a by-row call, needs the groups
    w12 = torch.tensor(_weights(rng, 27, 12, 16)).half().to(G.DEV)
    f12 = feat[:, :12].contiguous()
    assert torch.equal(ext.rule_conv(f12, w12, book, None, n), ext.rule_conv(f12, w12, ref_book, None, n))
    assert book.fwd.groups
    with torch.no_grad():
        book, _ = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3], weight=w)
    g = torch.tensor(rng.standard_normal((n, 16)), dtype=torch.float32).half().to(G.DEV)
    assert torch.equal(ext.rule_conv_d_weight(feat, g, book, None), ext.rule_conv_d_weight(feat, g, ref_book, None))
    assert book.fwd.groups
    with torch.no_grad():
        book, _ = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3], weight=w)
    r1, s1 = book.padded((2, 2))
    r2, s2 = ref_book.padded((2, 2))
    assert torch.equal(s1, s2) and torch.equal(r1, r2)


@pytest.mark.parametrize("p,shape,ic,oc,dtype", [(0.5, [24, 96, 16], 32, 32, torch.float16), (1.0, [18, 64, 16], 16, 64, torch.float16),
                                                 (0.08, [64, 256, 24], 32, 16, torch.float16), (0.5, [24, 96, 16], 16, 16, torch.float32),
                                                 (0.6, [24, 80, 16], 64, 32, torch.int8),
                                                 (0.5, [24, 96, 16], 16, 32, torch.float16), (0.5, [24, 96, 16], 8, 24, torch.bfloat16)])
def test_by_row_equals_groups_on_large_grids(monkeypatch, p, shape, ic, oc, dtype):
    """More than 1024 tiles (one wave per tile in the by-row kernel), dense to sparse, rows of 16, 32 and 64
    bytes (up to 32 bytes in 16-bit types: two kernel offsets per MFMA, forward or dgrad): same pairs as the grouped kernel, forward and dgrad (int8 equal; floating point to the path's tolerance:
    the two kernels add a row's products in different orders)."""
    from sphconv_amd import rulebook
    from sphconv_amd.rulebook import RuleBook
    rng = np.random.default_rng(int(p * 100) + ic)
    B = 8
    occ = rng.random((B, *shape)) < p
    idx = np.argwhere(occ).astype(np.int32)
    _, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    n = z_idx.shape[0]
    assert n > 1024 * 128
    zi, zp = G.t(z_idx), G.t(z_ptr)
    if dtype == torch.int8:
        feat = torch.tensor(rng.integers(-128, 128, (n, ic), dtype=np.int8)).to(G.DEV)
        w = torch.tensor(rng.integers(-128, 128, (27, ic, oc), dtype=np.int8)).to(G.DEV)
        scale = torch.tensor(((rng.random(oc) + 0.5) / 3000.0).astype(np.float32)).to(G.DEV)
        run = lambda book: ext.rule_conv_int8(feat, w, scale, book, None, n)
    else:
        feat = torch.tensor(rng.standard_normal((n, ic)), dtype=torch.float32).to(dtype).to(G.DEV)
        w = torch.tensor(_weights(rng, 27, ic, oc)).to(dtype).to(G.DEV)
        run = lambda book: ext.rule_conv(feat, w, book, None, n)
    out = {}
    for form, thr in (("groups", float("inf")), ("by_row", 0.0)):
        monkeypatch.setattr(rulebook, "BY_ROW_MIN_PAIRS", thr)
        book = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3])
        assert (book.fwd.tile_nbr is not None) == (form == "by_row")
        out[form] = run(book)
        if dtype != torch.int8:
            g = torch.tensor(rng.standard_normal((n, oc)), dtype=torch.float32).to(dtype).to(G.DEV) if form == "groups" else g
            wt = w.permute(0, 2, 1).contiguous()
            out[form + "_d"] = ext.rule_conv_d_feature(g, wt, book, None, None, n)
    G.assert_same_conv(out["groups"], out["by_row"])
    assert float(out["groups"].float().abs().mean()) > 0
    if dtype != torch.int8:
        G.assert_same_conv(out["groups_d"], out["by_row_d"])


@pytest.mark.parametrize("kernel,stride,padding,ic,oc,dtype", [([3, 3, 3], [2, 2, 2], [1, 1, 1], 32, 32, torch.float16),
                                                              ([3, 3, 3], [1, 2, 1], [1, 1, 1], 16, 32, torch.bfloat16),
                                                              ([2, 2, 2], [2, 2, 2], [0, 0, 0], 16, 16, torch.float32)])
def test_by_row_equals_groups_on_large_strided_grids(monkeypatch, kernel, stride, padding, ic, oc, dtype):
    """Strided layers with more than 1024 output tiles and 64-byte rows (the by-row kernel that stages the
    gathered rows in LDS, with footprints that do and do not fit its window, kernel volumes that are and
    are not a multiple of its phase of 9 offsets): forward on the book and dgrad on the transposed book
    agree with the grouped kernels to the path's tolerance, and the forward result matches the oracle's."""
    from sphconv_amd import rulebook
    from sphconv_amd.rulebook import RuleBook
    rng = np.random.default_rng(ic + oc)
    B, shape = 4, [32, 512, 32]
    occ = rng.random((B, *shape)) < 0.3
    idx = np.argwhere(occ).astype(np.int32)
    _, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    n = z_idx.shape[0]
    oshape = H.out_shape_of(shape, kernel, stride, padding)
    zi, zp = G.t(z_idx), G.t(z_ptr)
    kv = kernel[0] * kernel[1] * kernel[2]
    feat = torch.tensor(rng.standard_normal((n, ic)), dtype=torch.float32).to(dtype).to(G.DEV)
    w = torch.tensor(_weights(rng, kv, ic, oc)).to(dtype).to(G.DEV)
    wt = w.permute(0, 2, 1).contiguous()
    out = {}
    for form, thr in (("groups", float("inf")), ("by_row", 0.0)):
        monkeypatch.setattr(rulebook, "BY_ROW_MIN_PAIRS", thr)
        book = RuleBook.build(zi, zp, B, shape, oshape, kernel, stride, padding)
        m = book.out_rows
        assert m > 1024 * 128 and n > 1024 * 128
        assert (book.fwd.tile_nbr is not None) == (form == "by_row")
        out[form] = ext.rule_conv(feat, w, book, None, m)
        g = torch.tensor(rng.standard_normal((m, oc)), dtype=torch.float32).to(dtype).to(G.DEV) if form == "groups" else g
        out[form + "_d"] = ext.rule_conv_d_feature(g, wt, book, None, None, n)
    G.assert_same_conv(out["groups"], out["by_row"])
    G.assert_same_conv(out["groups_d"], out["by_row_d"])
    ora = O.get_rules(z_idx, z_ptr, B, shape, oshape, kernel, stride, padding, n_max=512)
    oz_idx, oz_ptr, rules, rule_size, dropped = ora
    assert dropped == 0 and oz_idx.shape[0] == m
    want = O.rule_conv(feat.float().cpu().numpy(), w.float().cpu().numpy(), rules, rule_size, m)
    got = out["by_row"].float().cpu().numpy()
    tol = {torch.float16: 2.0 ** -9, torch.bfloat16: 2.0 ** -7, torch.float32: 1e-5}[dtype]
    assert (np.abs(got - want) <= tol * np.abs(want) + 1e-3).all()
    assert np.abs(want).mean() > 1e-2


def test_forward_only_books_go_by_rows_from_a_lower_density(monkeypatch):
    """A book built with its layer's weight while no gradient is recorded leaves its groups out, so it keeps
    the pairs by row from 0.65 x the usual estimate of pairs per row; any other book of the same tensor
    stays grouped below the usual threshold.  Same results either way."""
    from sphconv_amd import rulebook
    from sphconv_amd.rulebook import RuleBook
    monkeypatch.setattr(rulebook, "BY_ROW_MIN_PAIRS", 10.0)
    rng = np.random.default_rng(77)
    B, shape = 2, [16, 64, 16]
    occ = rng.random((B, *shape)) < 0.3          # estimate 27 * 0.3 = 8.1 pairs per row
    idx = np.argwhere(occ).astype(np.int32)
    _, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    n = z_idx.shape[0]
    zi, zp = G.t(z_idx), G.t(z_ptr)
    feat = torch.tensor(rng.standard_normal((n, 32)), dtype=torch.float32).half().to(G.DEV)
    w = torch.tensor(_weights(rng, 27, 32, 32)).half().to(G.DEV)
    with torch.no_grad():
        fwd_only, packed = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3], weight=w)
    assert 10.0 * rulebook.BY_ROW_FORWARD_ONLY <= fwd_only._pairs_per_row(False) < 10.0
    assert fwd_only.fwd.tile_nbr is not None and not fwd_only.fwd.groups
    with torch.enable_grad():
        training, _ = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3], weight=w)
    plain = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3])
    for book in (training, plain):
        assert book.fwd.tile_nbr is None and book.fwd.groups
    a = ext.rule_conv(feat, w, fwd_only, None, n, packed=packed)
    b = ext.rule_conv(feat, w, plain, None, n)
    G.assert_same_conv(a, b)
    assert float(a.float().abs().mean()) > 0
    sparse = rng.random((B, *shape)) < 0.2       # estimate 5.4: below both thresholds
    _, z_idx2, z_ptr2, _ = H.csr_from_indices(np.argwhere(sparse).astype(np.int32), B, shape)
    with torch.no_grad():
        book, _ = RuleBook.build_subm(G.t(z_idx2), G.t(z_ptr2), B, shape, [3, 3, 3], weight=w)
    assert book.fwd.tile_nbr is None and book.fwd.groups


def test_wgrad_many_slots_equals_sum_over_samples():
    """Rules never cross batch samples, so d_weight of a batch is the sum of the samples' d_weights.  With 14
    scans of the configuration-3 grid (2.2 M rows, 17 000 tiles) the slot reduction walks more than 1024
    partial slots per offset, i.e. more than one pass of its flag words; each sample alone needs 80."""
    from sphconv_amd.rulebook import RuleBook
    B = 14
    d = make_config(3, seed=3, batch=B)
    shape = d["spatial_shape"]
    n = int(d["z_idx"].shape[0])
    assert n > 128 * 64 * 256                       # more than 256 chunks of 64 tiles: > 1024 slots per offset
    ic = oc = 16
    gen = torch.Generator(device=G.DEV).manual_seed(9)
    feat = torch.randn((n, ic), device=G.DEV, generator=gen).half()
    g = torch.randn((n, oc), device=G.DEV, generator=gen).half()
    zi, zp = G.t(d["z_idx"]), G.t(d["z_ptr"])
    book = RuleBook.build_subm(zi, zp, B, shape, [3, 3, 3])
    whole = ext.rule_conv_d_weight(feat, g, book, None).float()
    ends = d["z_ptr"].reshape(B, -1)[:, -1].astype(np.int64)
    starts = np.concatenate([[0], ends[:-1]])
    parts = torch.zeros_like(whole)
    pairs = 0
    for b in range(B):
        s, e = int(starts[b]), int(ends[b])
        zp_b = G.t((d["z_ptr"][b:b + 1] - s).astype(np.int32))
        bk = RuleBook.build_subm(zi[s:e].contiguous(), zp_b, 1, shape, [3, 3, 3])
        parts += ext.rule_conv_d_weight(feat[s:e].contiguous(), g[s:e].contiguous(), bk, None).float()
        pairs += bk.num_pairs()
    assert pairs == book.num_pairs()
    # every part was rounded to fp16 once, the whole once; the sums run over up to 2.2 M products (centre offset)
    scale = float(whole.abs().max())
    assert float((whole - parts).abs().max()) <= 2.0 ** -9 * scale * np.sqrt(B) + 1e-2


def test_fp32_master_weight_gets_an_fp32_gradient():
    """fp16 features with an fp32 weight (mixed-precision training): the weight's gradient is the fp32
    reduction itself, never rounded to, or overflowing in, fp16."""
    from sphconv_amd.functional import ConvFunction
    case = _random_case(77, True)
    rng = np.random.default_rng(5)
    n = case["sidx"].shape[0]
    # values whose sums over a neighbourhood leave fp16's range: a 16-bit d_weight would be inf
    feat = G.t(rng.standard_normal((n, 16)).astype(np.float32) * 60).half().requires_grad_(True)
    w = G.t(_weights(rng, 27, 16, 32)).requires_grad_(True)
    out = ConvFunction.apply(feat, w, case["book"], None, [1, 1], n)
    assert out.dtype == torch.float16
    up = G.t(rng.standard_normal((n, 32)).astype(np.float32) * 60).half()
    out.backward(up)
    assert w.grad.dtype == torch.float32 and torch.isfinite(w.grad).all()
    wide = ext.rule_conv_d_weight(feat.detach(), up, case["book"], None, torch.float32)
    assert torch.equal(w.grad, wide)
    assert wide.abs().max() > 65504          # the case does leave fp16's range
    narrow = ext.rule_conv_d_weight(feat.detach(), up, case["book"], None)
    assert torch.isinf(narrow).any()


@pytest.mark.parametrize("rows", [(1 << 24) - 64, (1 << 24) + 4096], ids=["just-below-2GiB", "above-2GiB"])
def test_feature_arrays_around_two_gib(rows):
    """The one-wave-per-tile kernel addresses the features through a buffer descriptor with 31-bit byte offsets
    made by a 24-bit multiply: arrays below 2 GiB and 2^24 rows take it (checked with a book that gathers from
    the array's last rows, where the offsets are largest: a wrong offset reads zeros, it cannot fault); an array
    of 2 GiB or more goes to the general kernel, whose 64-bit addressing (and the by-row kernels') is checked
    the same way."""
    case = _random_case(91, True)
    rng = np.random.default_rng(3)
    n = case["sidx"].shape[0]
    feat = rng.standard_normal((n, 64)).astype(np.float32)
    w = _weights(rng, 27, 64, 64)
    book = case["book"]
    want = _oracle_fwd(case, torch.tensor(feat).half().float().numpy(), torch.tensor(w).half().float().numpy())
    small = ext.rule_conv(G.t(feat).half(), G.t(w).half(), book, None, n)
    np.testing.assert_allclose(small.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)
    base = rows - n                               # rows x 128 bytes = 2 GiB -/+ a little
    big = torch.zeros((rows, 64), dtype=torch.float16, device=G.DEV)
    big[base:] = G.t(feat).half()
    tables = [book.fwd.grp_gather] + ([book.fwd.tile_nbr] if book.fwd.by_row else [])   # both forms name gathered rows
    keep = [t.clone() for t in tables]
    try:
        for t, k in zip(tables, keep):
            t.copy_(torch.where(k >= 0, k + base, k))
        packed = ext._packed_weight(G.t(w).half(), False)
        out = ext._apply(big, packed, 64, 64, book.fwd)
    finally:
        for t, k in zip(tables, keep):
            t.copy_(k)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(out.float(), small.float(), rtol=1e-3, atol=1e-3)
