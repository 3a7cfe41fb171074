"""GPU parity of rule generation against the CPU oracle (bit-exact).

Every case builds the rule book through the C ABI (sph_rules_build,
sph_outcoords_*), decodes it on the host and compares the set of
(k, input row, output row) triples, the output coordinates and -- through
sph_rules_to_padded_* -- the reference-format tensors with the oracle's."""
import numpy as np
import pytest
import torch

import helpers as H
import gpu_helpers as G
from oracle import oracle as O
from sphconv_amd import sphconv_cuda as ext
from sphconv_amd.rulebook import RuleBook
from sphconv_amd.synth import make_config

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("pair_form")]
CASES = H.load_ref_cases()


def _rule_calls():
    out = []
    for tc in CASES:
        if tc["file"] not in ("test/test_rules.py", "test/test_conv.py", "test/test_module.py"):
            continue
        for c in tc["calls"]:
            a = c["args"]
            if "spatial_shape_DWH" not in a and tc["file"] != "test/test_rules.py":
                continue
            out.append(pytest.param(tc["tensors"][c["coords"]], a,
                                    id="%s:%d" % (tc["file"].split("/")[-1], c["line"])))
    return out


def _check(case, tile=(2, 2)):
    book, ora = case["book"], case["oracle"]
    oz_idx, oz_ptr, rules, rule_size, dropped = ora
    assert dropped == 0
    # output coordinates
    assert book.out_rows == oz_idx.shape[0]
    assert np.array_equal(book.oz_idx.cpu().numpy(), oz_idx)
    assert np.array_equal(book.oz_ptr.cpu().numpy(), np.asarray(oz_ptr).reshape(book.oz_ptr.shape))
    # forward book == oracle pairs; transposed book == the same pairs, owner/gather swapped
    want = G.oracle_triples(rules, rule_size)
    got = G.book_triples(book.fwd)
    assert np.array_equal(got, want)
    got_t = G.book_triples(book.transposed())
    assert np.array_equal(got_t, G.oracle_triples(rules, rule_size, swap=True))
    assert book.num_pairs() == want.shape[0]
    # the same pairs by stationary row, where the book keeps that form
    for buf, tri in ((book.fwd, want), (book.transposed(), got_t)):
        rows = G.by_row_triples(buf)
        assert rows is None or np.array_equal(rows, tri)
    # reference-format tensors
    p_rules, p_size = book.padded(tile)
    assert np.array_equal(p_size.cpu().numpy(), rule_size)
    pr = p_rules.cpu().numpy()
    n = min(pr.shape[3], rules.shape[3])
    assert pr.shape[3] >= rule_size.max(initial=0)
    assert np.array_equal(pr[..., :n], rules[..., :n])
    assert (pr[..., n:] == -1).all()
    # and back: padded -> book
    rb2 = RuleBook.from_padded(p_rules, p_size, book.in_rows, book.out_rows)
    assert np.array_equal(G.book_triples(rb2.fwd), want)
    assert np.array_equal(G.book_triples(rb2.transposed()), got_t)


@pytest.mark.parametrize("coords,args", _rule_calls())
def test_reference_lists(coords, args):
    subm = bool(args.get("subm", False))
    B = args.get("batch_size", 1)
    shape = args.get("spatial_shape_DWH", [8, 8, 8])
    kernel = args.get("kernel_size", [3, 3, 3])
    stride = args.get("stride", [2, 2, 2])
    padding = args.get("padding", [1, 1, 1])
    idx = H.dup_with_batch_idx(coords, B)
    if not subm and min(H.out_shape_of(shape, kernel, stride, padding)) <= 0:
        pytest.skip("empty output grid")
    _check(G.build_case(idx, B, shape, kernel, stride, padding, subm))


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("subm,kernel,stride,padding", [
    (True, [3, 3, 3], [1, 1, 1], [1, 1, 1]),
    (True, [2, 2, 2], [1, 1, 1], [1, 1, 1]),
    (True, [1, 3, 5], [1, 1, 1], [0, 1, 2]),
    (False, [3, 3, 3], [2, 2, 2], [1, 1, 1]),
    (False, [3, 2, 3], [2, 1, 2], [1, 0, 1]),
    (False, [2, 2, 2], [2, 2, 2], [0, 0, 0]),
    (False, [3, 3, 3], [1, 1, 1], [0, 0, 0]),
    (False, [4, 4, 4], [3, 2, 1], [2, 1, 0]),
    (False, [3, 3, 3], [1, 2, 3], [1, 1, 1]),   # a stride along S2 that is no power of two: the division path
    (False, [3, 3, 5], [4, 4, 4], [1, 1, 2]),
    (True, [5, 5, 5], [1, 1, 1], [2, 2, 2]),      # kernel volume 125: the neighbour table needs 68 KB of LDS
])
def test_random_grids(seed, subm, kernel, stride, padding):
    rng = np.random.default_rng(seed)
    B, shape = 3, [9, 37, 21]
    occ = rng.random((B, *shape)) < (0.05, 0.3, 0.9)[seed]
    idx = np.argwhere(occ).astype(np.int32)
    _check(G.build_case(idx, B, shape, kernel, stride, padding, subm), tile=(2, 2))


@pytest.mark.parametrize("B,shape,n,subm,kernel,stride,padding", [
    (2, [509, 1021, 5], 60000, True, [3, 3, 3], [1, 1, 1], [1, 1, 1]),     # 1.04 M columns, prime line lengths
    (1, [3, 65537, 9], 40000, True, [3, 3, 3], [1, 1, 1], [1, 1, 1]),      # a line longer than 2^16 columns
    (5, [127, 129, 33], 50000, False, [3, 3, 3], [2, 2, 2], [1, 1, 1]),
    (3, [1, 131071, 4], 30000, False, [1, 3, 3], [1, 2, 1], [0, 1, 1]),    # one line per sample, 2^17 - 1 columns
])
def test_large_grids_with_odd_line_lengths(B, shape, n, subm, kernel, stride, padding):
    """A row's column index is split into (batch, S0, S1) with division constants made on the host
    (multiply-high and shifts): line lengths that are no powers of two, large column indices, the last
    columns of the last sample occupied.  Pairs against the oracle's, forward and transposed."""
    rng = np.random.default_rng(shape[1])
    cells = B * shape[0] * shape[1] * shape[2]
    lin = rng.choice(cells - 64, size=n, replace=False)
    lin = np.concatenate([lin, np.arange(cells - 64, cells)])          # the grid's very last cells
    idx = np.stack(np.unravel_index(lin, (B, *shape)), axis=1).astype(np.int32)
    _check(G.build_case(idx, B, shape, kernel, stride, padding, subm), tile=(2, 2))


def test_deep_axis_more_than_64_bins():
    """S2 = 200 > 64 exercises the multi-pass output-bin masks."""
    rng = np.random.default_rng(3)
    B, shape = 2, [5, 6, 200]
    occ = rng.random((B, *shape)) < 0.1
    idx = np.argwhere(occ).astype(np.int32)
    _check(G.build_case(idx, B, shape, [3, 3, 3], [2, 2, 2], [1, 1, 1], False))
    _check(G.build_case(idx, B, shape, [3, 3, 3], [1, 1, 1], [1, 1, 1], True))


def test_empty_and_single():
    z_ptr = torch.zeros((2, 4, 4), dtype=torch.int32, device=G.DEV)
    z_idx = torch.zeros((0,), dtype=torch.int32, device=G.DEV)
    b = RuleBook.build_subm(z_idx, z_ptr, 2, [4, 4, 4], [3, 3, 3])
    assert b.num_pairs() == 0 and b.fwd.ntiles == 0
    b = RuleBook.build(z_idx, z_ptr, 2, [4, 4, 4], [2, 2, 2], [3, 3, 3], [2, 2, 2], [1, 1, 1])
    assert b.out_rows == 0 and int(b.oz_ptr.abs().sum()) == 0
    # empty samples and long empty column runs between occupied ones
    idx = np.array([[0, 0, 0, 1], [3, 63, 511, 30]], np.int32)
    _check(G.build_case(idx, 4, [64, 512, 32], [3, 3, 3], [1, 1, 1], [1, 1, 1], True))
    _check(G.build_case(idx, 4, [64, 512, 32], [3, 3, 3], [2, 2, 2], [1, 1, 1], False))


def test_dense_block_fills_every_offset():
    idx = np.array([[0, a, b, c] for a in range(6) for b in range(7) for c in range(8)], np.int32)
    case = G.build_case(idx, 1, [6, 7, 8], [3, 3, 3], [1, 1, 1], [1, 1, 1], True)
    _check(case)
    assert case["book"].num_pairs() == int(case["oracle"][3].sum())


@pytest.mark.parametrize("cfg", [1, 2, 3, 5])
def test_benchmark_configs_full_size(cfg):
    """BASELINE configurations at full size, bit-exact against the oracle."""
    d = make_config(cfg, seed=0)
    subm = cfg != 3
    kernel = [3, 3, 3]
    stride, padding = ([1, 1, 1], [1, 1, 1]) if subm else ([2, 2, 2], [1, 1, 1])
    shape, B = d["spatial_shape"], d["batch"]
    oshape = shape if subm else H.out_shape_of(shape, kernel, stride, padding)
    zi, zp = G.t(d["z_idx"]), G.t(d["z_ptr"])
    book = (RuleBook.build_subm(zi, zp, B, shape, kernel) if subm else
            RuleBook.build(zi, zp, B, shape, oshape, kernel, stride, padding))
    fn = O.get_rules_subm if subm else O.get_rules
    oz_idx, oz_ptr, rules, rule_size, dropped = fn(d["z_idx"], d["z_ptr"], B, shape, oshape, kernel,
                                                   stride, padding, (1, 1, 1), (2, 2), n_max=None)
    assert np.array_equal(book.oz_idx.cpu().numpy(), oz_idx)
    assert np.array_equal(book.oz_ptr.cpu().numpy().ravel(), np.asarray(oz_ptr).ravel())
    if dropped == 0:
        want = G.oracle_triples(rules, rule_size)
        assert np.array_equal(G.book_triples(book.fwd), want)
        p_rules, p_size = book.padded((2, 2))
        assert np.array_equal(p_size.cpu().numpy(), rule_size)
    else:
        # the reference's heuristic tile_n_max overflows on this input: compare counts only
        assert book.num_pairs() == int(rule_size.sum())
    # size-independent properties
    got = G.book_triples(book.fwd)
    if subm:
        n = zi.shape[0]
        centre = got[got[:, 0] == 13]
        assert centre.shape[0] == n and (centre[:, 1] == centre[:, 2]).all()
        back = got[:, [0, 2, 1]].copy()
        back[:, 0] = 26 - back[:, 0]
        order = np.lexsort((back[:, 2], back[:, 0]))
        assert np.array_equal(back[order], got)            # pair symmetry k <-> 26-k
    for k in range(27):
        o = got[got[:, 0] == k][:, 2]
        assert np.unique(o).shape[0] == o.shape[0]         # per-k output rows unique


def test_extension_functions_match_reference_signatures():
    idx = np.array(CASES[2]["tensors"]["indices"], np.int32)
    idx = H.dup_with_batch_idx(idx, 2)
    feat = np.random.default_rng(0).standard_normal((idx.shape[0], 4)).astype(np.float32)
    f, z_idx, z_ptr, perm = ext.init_tensor(G.t(feat), G.t(idx), 2, [8, 9, 9])
    f2, z2, p2, perm2 = O.init_tensor(feat, idx, 2, [8, 9, 9])
    assert np.array_equal(f.cpu().numpy(), f2) and np.array_equal(z_idx.cpu().numpy(), z2)
    assert np.array_equal(z_ptr.cpu().numpy(), p2) and np.array_equal(perm.cpu().numpy(), perm2)
    r = ext.get_rules_subm(z_idx, z_ptr, 2, [8, 9, 9], [8, 9, 9], [3, 3, 3], [1, 1, 1], [1, 1, 1],
                           [1, 1, 1], [2, 2])
    assert r[0] is z_idx and r[1] is z_ptr
    _, _, rules, rule_size, _ = O.get_rules_subm(z2, p2, 2, [8, 9, 9], [8, 9, 9], [3, 3, 3], [1, 1, 1],
                                                 [1, 1, 1])
    assert np.array_equal(r[3].cpu().numpy(), rule_size)
    n = rules.shape[3]
    assert np.array_equal(r[2].cpu().numpy()[..., :n], rules)
    with pytest.raises(ValueError):
        ext.init_tensor(G.t(np.concatenate([feat, feat[:1]])), G.t(np.concatenate([idx, idx[:1]])), 2, [8, 9, 9])
    bad = idx.copy(); bad[0, 3] = 99
    with pytest.raises(ValueError):
        ext.init_tensor(G.t(feat), G.t(bad), 2, [8, 9, 9])
    # 50 000 copies of one coordinate: reported as duplicates without walking the column once per copy
    many = np.repeat(idx[:1], 50000, axis=0)
    with pytest.raises(ValueError, match="duplicate"):
        ext.init_tensor(G.t(np.zeros((50000, 2), np.float32)), G.t(many), 2, [8, 9, 9])
    # the same mistakes on a grid deep enough for the bitmap path
    deep = idx.copy(); deep[:, 3] = deep[:, 3] * 30 + 7
    ext.init_tensor(G.t(feat), G.t(deep), 2, [8, 9, 300])
    with pytest.raises(ValueError, match="duplicate"):
        ext.init_tensor(G.t(np.concatenate([feat, feat[:1]])), G.t(np.concatenate([deep, deep[:1]])), 2, [8, 9, 300])
    bad = deep.copy(); bad[0, 3] = 300
    with pytest.raises(ValueError):
        ext.init_tensor(G.t(feat), G.t(bad), 2, [8, 9, 300])
    with pytest.raises(ValueError, match="duplicate"):
        ext.init_tensor(G.t(np.zeros((50000, 2), np.float32)), G.t(np.repeat(deep[:1], 50000, axis=0)), 2, [8, 9, 300])


@pytest.mark.parametrize("B,shape,n", [(1, (64, 512, 32), 40000), (3, (7, 5, 3), 50), (2, (2048, 2048, 1024), 3000),
                                       (1, (4, 4, 4), 0), (1, (1, 1, 1), 1), (2, (8, 8, 64), 6000),
                                       (1, (16, 16, 128), 20000), (1, (16, 16, 129), 20000), (1, (3, 3, 200), 0),
                                       (1, (1024, 1024, 16), 150000), (2, (512, 300, 130), 90000),
                                       (1, (8, 8, 300), 15000), (2, (5, 7, 64 * 3), 6000)])
def test_init_tensor_sizes(B, shape, n):
    """COO -> compressed layout at sizes whose cells need more than 32 bits, one cell, no voxel
    at all, long fibers, either side of the depth (128 bins) from which a row's rank comes from its column's
    bitmap instead of a walk over the column's rows, deep grids that are nearly full (columns of hundreds of rows),
    a deep grid whose bitmap would exceed the library's limit (2048 x 2048 x 1024: ranked by the walk), and column
    counts whose scan looks back over more than 64 workgroups (1M and 307k columns); checked against the oracle
    and against the defining invariants."""
    rng = np.random.default_rng(B * 1000 + n)
    cells = B * shape[0] * shape[1] * shape[2]
    lin = np.unique(rng.integers(0, cells, size=n, dtype=np.int64))[:n] if n else np.zeros(0, np.int64)
    rng.shuffle(lin)
    idx = np.stack(np.unravel_index(lin, (B,) + tuple(shape)), axis=1).astype(np.int32).reshape(-1, 4)
    feat = rng.standard_normal((idx.shape[0], 5)).astype(np.float32)
    f, z_idx, z_ptr, perm = ext.init_tensor(G.t(feat), G.t(idx), B, list(shape))
    f, z_idx, z_ptr, perm = f.cpu().numpy(), z_idx.cpu().numpy(), z_ptr.cpu().numpy(), perm.cpu().numpy()
    # invariants: inclusive counts per column, ascending S2 inside a fiber, rows follow the permutation
    col = (idx[:, 0].astype(np.int64) * shape[0] + idx[:, 1]) * shape[1] + idx[:, 2]
    counts = np.bincount(col, minlength=B * shape[0] * shape[1])
    assert np.array_equal(z_ptr.reshape(-1), np.cumsum(counts))
    assert np.array_equal(np.sort(perm), np.arange(idx.shape[0]))
    assert np.array_equal(f[perm], feat) and np.array_equal(z_idx[perm], idx[:, 3])
    order = np.argsort(lin, kind="stable")
    assert np.array_equal(perm[order], np.arange(idx.shape[0]))
    if cells < 1 << 24:
        f2, z2, p2, perm2 = O.init_tensor(feat, idx, B, list(shape))
        assert np.array_equal(f, f2) and np.array_equal(z_idx, z2) and np.array_equal(z_ptr, p2)
        assert np.array_equal(perm, perm2)
    # backward of the row move
    g = rng.standard_normal(f.shape).astype(np.float32)
    back = ext.init_tensor_backward(G.t(g), G.t(perm)).cpu().numpy()
    assert np.array_equal(back, g[perm])


def test_unsorted_long_fibers_take_the_general_join():
    """Long fibers are joined through per-column bin masks, which needs them in ascending S2 order
    (as init_tensor and the strided rule generation emit them); a tensor whose fibers are in another
    order (legal in the reference: tensor.cu:61-65 leaves the order to the atomics) must give the
    same pairs through the general join."""
    rng = np.random.default_rng(11)
    B, shape = 2, [6, 9, 16]
    occ = rng.random((B, *shape)) < 0.6
    idx = np.argwhere(occ).astype(np.int32)
    _, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    assert z_idx.shape[0] >= 4 * B * shape[0] * shape[1]
    ends = z_ptr.reshape(-1)
    starts = np.concatenate([[0], ends[:-1]])
    z_rev = z_idx.copy()
    for s, e in zip(starts, ends):
        z_rev[s:e] = z_idx[s:e][::-1]
    assert not np.array_equal(z_rev, z_idx)
    for zi in (z_idx, z_rev):
        book = RuleBook.build_subm(G.t(zi), G.t(z_ptr), B, shape, [3, 3, 3])
        _, _, rules, rule_size, dropped = O.get_rules_subm(zi, z_ptr, B, shape, shape, [3, 3, 3], [1, 1, 1], [1, 1, 1],
                                                           (1, 1, 1), (2, 2), n_max=256)
        assert dropped == 0
        assert np.array_equal(G.book_triples(book.fwd), G.oracle_triples(rules, rule_size))
        assert np.array_equal(G.book_triples(book.transposed()), G.oracle_triples(rules, rule_size, swap=True))


def test_outcoords_total_is_optional():
    """sph_outcoords_count writes the output row count to *total_dev when given one; either way the count is
    the last element of the scanned oz_ptr.  The scratch may hold anything on entry (the call clears the state
    of the scan across workgroups itself), so one scratch serves call after call."""
    import ctypes as C
    from sphconv_amd import _lib as L
    rng = np.random.default_rng(5)
    B, shape, out_shape = 2, [9, 20, 12], [5, 10, 6]
    idx = np.argwhere(rng.random((B, *shape)) < 0.2).astype(np.int32)
    _, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    zi, zp = G.t(z_idx), G.t(z_ptr)
    lib = L.lib()
    g = L.make_geom(B, shape, out_shape, [3, 3, 3], [2, 2, 2], [1, 1, 1], [1, 1, 1])
    n = lib.sph_outcoords_scratch_ints(C.byref(g))
    ns = lib.sph_outcoords_state_ints(C.byref(g))
    assert 0 < ns <= n
    ptrs = []
    scratch = torch.full((n + (n & 1),), -1, dtype=torch.int32, device="cuda:0")    # garbage on entry
    for with_total in (True, False):
        oz_ptr = torch.empty((B, out_shape[0], out_shape[1]), dtype=torch.int32, device="cuda:0")
        total = torch.full((1,), -7, dtype=torch.int32, device="cuda:0")
        L.check(lib.sph_outcoords_count(L.ptr(zi), L.ptr(zp), int(zi.shape[0]), C.byref(g), L.ptr(oz_ptr),
                                        L.ptr(scratch), L.ptr(total) if with_total else None, L.stream()))
        torch.cuda.synchronize()
        assert int(total.item()) == (int(oz_ptr.view(-1)[-1].item()) if with_total else -7)
        ptrs.append(oz_ptr.cpu().numpy())
    assert np.array_equal(ptrs[0], ptrs[1])
    book = RuleBook.build(zi, zp, B, shape, out_shape, [3, 3, 3], [2, 2, 2], [1, 1, 1])
    assert np.array_equal(book.oz_ptr.cpu().numpy(), ptrs[0]) and book.out_rows == int(ptrs[0].reshape(-1)[-1])


@pytest.mark.parametrize("shape,p", [([40, 700, 20], 0.02), ([64, 1024, 70], 0.05), ([3, 21, 9], 0.5),
                                     ([500, 599, 8], 0.01), ([10, 30, 400], 0.05), ([12, 20, 250], 0.05),
                                     ([6, 20, 1100], 0.02), ([900, 700, 4], 0.01)])
def test_outcoords_scan_over_many_workgroups(shape, p):
    """Per-column counts and their one-pass scan (tiles of 2048 columns that look back over their
    predecessors): grids of one tile, of tens and of more than 64 tiles (several look-back windows), ragged
    ends, and output columns of 125, 200 and 550 bins (two and four masks per column kept; none beyond 512
    bins), twice in a row on the same scratch, against numpy's cumsum and the active set of a dense convolution."""
    import ctypes as C
    from sphconv_amd import _lib as L
    rng = np.random.default_rng(shape[1])
    B = 3
    idx = np.argwhere(rng.random((B, *shape)) < p).astype(np.int32)
    _, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    out_shape = H.out_shape_of(shape, [3, 3, 3], [2, 2, 2], [1, 1, 1])
    occ = np.zeros((B, *shape), np.float32)
    occ[tuple(idx.T)] = 1
    act = torch.nn.functional.conv3d(torch.tensor(occ)[:, None], torch.ones((1, 1, 3, 3, 3)), stride=2, padding=1)[:, 0] != 0
    want = np.cumsum(act.sum(3).numpy().reshape(-1)).astype(np.int32)
    lib = L.lib()
    g = L.make_geom(B, shape, out_shape, [3, 3, 3], [2, 2, 2], [1, 1, 1], [1, 1, 1])
    n = lib.sph_outcoords_scratch_ints(C.byref(g))
    scratch = torch.empty(n + (n & 1), dtype=torch.int32, device="cuda:0")
    zi, zp = G.t(z_idx), G.t(z_ptr)
    for _ in range(2):
        oz_ptr = torch.full((B, out_shape[0], out_shape[1]), -1, dtype=torch.int32, device="cuda:0")
        total = torch.zeros(1, dtype=torch.int32).pin_memory()
        L.check(lib.sph_outcoords_count(L.ptr(zi), L.ptr(zp), int(zi.shape[0]), C.byref(g), L.ptr(oz_ptr),
                                        L.ptr(scratch), total.data_ptr(), L.stream()))
        torch.cuda.current_stream().synchronize()
        assert int(total[0]) == int(want[-1])            # written by the kernel to pinned host memory
        assert np.array_equal(oz_ptr.cpu().numpy().reshape(-1), want)
        # the bins themselves: from the masks the count kernel kept (up to 512 bins) or from a second walk
        m = int(total[0])
        oz_idx = torch.full((max(m, 1),), -1, dtype=torch.int32, device="cuda:0")
        L.check(lib.sph_outcoords_fill(L.ptr(zi), L.ptr(zp), int(zi.shape[0]), C.byref(g), L.ptr(scratch),
                                       L.ptr(oz_ptr), L.ptr(oz_idx), m, None, L.stream()))
        assert np.array_equal(oz_idx.cpu().numpy()[:m], np.nonzero(act.numpy())[3].astype(np.int32))
