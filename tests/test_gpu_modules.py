"""Module-level GPU tests: the reference's Python API (SparseConvTensor, Conv3d /
SubMConv3d, Sequential, RangeVoxel, autograd) against torch's dense conv3d."""
import numpy as np
import pytest
import torch

import helpers as H
import gpu_helpers as G
import sphconv_amd as sphconv
from oracle import oracle as O
from sphconv_amd.synth import make_config

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("pair_form")]


def _inputs(seed, B, shape, C, p=0.2, dtype=torch.float32):
    rng = np.random.default_rng(seed)
    occ = rng.random((B, *shape)) < p
    idx = np.argwhere(occ).astype(np.int32)
    idx = idx[rng.permutation(idx.shape[0])]
    feat = rng.standard_normal((idx.shape[0], C)).astype(np.float32)
    return idx, feat


def test_dense_roundtrip_and_grads():
    """Reference test_grad.py:144-185: scaling dense cells by 2 and 3 gives grads 2 and 3."""
    idx, feat = _inputs(0, 2, [5, 6, 7], 3)
    f = G.t(feat).requires_grad_(True)
    x = sphconv.SparseConvTensor(f, [5, 6, 7], 2, indices=G.t(idx))
    dense = x.dense()
    assert list(dense.shape) == [2, 3, 5, 6, 7]
    want = H.dense_from_rows(feat, idx, 2, [5, 6, 7], torch.float32)
    assert torch.equal(dense.detach().cpu(), want)
    scale = torch.ones_like(dense)
    scale[0] = 2.0
    scale[1] = 3.0
    (dense * scale).sum().backward()
    g = f.grad.cpu().numpy()
    assert np.array_equal(g[idx[:, 0] == 0], np.full_like(g[idx[:, 0] == 0], 2.0))
    assert np.array_equal(g[idx[:, 0] == 1], np.full_like(g[idx[:, 0] == 1], 3.0))


@pytest.mark.parametrize("subm,stride,padding", [(True, 1, 1), (False, 2, 1), (False, 1, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_conv_module_matches_dense_autograd(subm, stride, padding, dtype):
    B, shape, ic, oc = 2, [8, 12, 10], 8, 16
    idx, feat = _inputs(1, B, shape, ic)
    cls = sphconv.SubMConv3d if subm else sphconv.SparseConv3d
    conv = cls(ic, oc, 3, stride=stride, padding=padding, bias=False).to(G.DEV).to(dtype)
    f = G.t(feat).to(dtype).requires_grad_(True)
    x = sphconv.SparseConvTensor(f, shape, B, indices=G.t(idx))
    y = conv(x)
    dense_y = y.dense()
    # dense reference in float64 on the same (rounded) values
    w64 = conv.weight.detach().double().cpu().requires_grad_(True)
    f64 = f.detach().double().cpu().requires_grad_(True)
    c = torch.as_tensor(idx, dtype=torch.long)
    d_in = torch.zeros((B, *shape, ic), dtype=torch.float64).index_put((c[:, 0], c[:, 1], c[:, 2], c[:, 3]), f64)
    ref = torch.nn.functional.conv3d(d_in.permute(0, 4, 1, 2, 3), w64.permute(4, 3, 0, 1, 2), None, stride, padding)
    if subm:
        mask = H.dense_from_rows(np.ones((idx.shape[0], 1)), idx, B, shape)
        ref = ref * mask
    tol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=2e-3)
    torch.testing.assert_close(dense_y.detach().double().cpu(), ref.detach(), **tol)
    up = torch.randn(ref.shape, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    if subm:
        up = up * mask
    else:
        up = up * (ref.detach().abs().sum(1, keepdim=True) != 0)      # grads only at active outputs
    (ref * up).sum().backward()
    (dense_y * up.to(G.DEV).to(dtype)).sum().backward()
    gtol = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(f.grad.double().cpu(), f64.grad, **gtol)
    torch.testing.assert_close(conv.weight.grad.double().cpu(), w64.grad, **gtol)


def test_sequential_rule_reuse_and_plain_modules():
    B, shape = 2, [8, 16, 12]
    idx, feat = _inputs(2, B, shape, 4)
    net = sphconv.SparseSequential(
        sphconv.SubMConv3d(4, 8, 3, indice_key="s1"),
        torch.nn.BatchNorm1d(8), torch.nn.ReLU(),
        sphconv.SubMConv3d(8, 8, 3, indice_key="s1"),
        torch.nn.BatchNorm1d(8), torch.nn.ReLU(),
        sphconv.SparseConv3d(8, 16, 3, stride=2, padding=1),
    ).to(G.DEV).eval()
    x = sphconv.SparseConvTensor(G.t(feat), shape, B, indices=G.t(idx))
    with torch.no_grad():
        y = net(x)
    assert "s1" in x.rule_cache and net[0].rule_book is net[3].rule_book
    assert [y.D, y.W, y.H] == [4, 8, 6] and y.feature.shape[1] == 16
    # dense re-computation
    with torch.no_grad():
        d = x.dense().cpu().double()
        mask = (H.dense_from_rows(np.ones((idx.shape[0], 1)), idx, B, shape) != 0).double()
        for i in (0, 3):
            w = net[i].weight.detach().cpu().double().permute(4, 3, 0, 1, 2)
            d = torch.nn.functional.conv3d(d, w, None, 1, 1) * mask
            bn = net[i + 1]
            s = (bn.weight / torch.sqrt(bn.running_var + bn.eps)).cpu().double()
            sh = (bn.bias - bn.running_mean * bn.weight / torch.sqrt(bn.running_var + bn.eps)).cpu().double()
            d = torch.relu(d * s[None, :, None, None, None] + sh[None, :, None, None, None]) * mask
        w = net[6].weight.detach().cpu().double().permute(4, 3, 0, 1, 2)
        d = torch.nn.functional.conv3d(d, w, None, 2, 1)
    torch.testing.assert_close(y.dense().cpu().double(), d, rtol=1e-4, atol=1e-5)
    assert net[0].rule_size.shape == (4 * 8, 27)


def test_rangevoxel_bridge():
    B, H_, W_, D_, C = 2, 6, 9, 11, 3
    idx, feat = _inputs(3, B, [H_, W_, D_], C, p=0.3)
    x = sphconv.SparseConvTensor(G.t(feat), [H_, W_, D_], B, indices=G.t(idx))
    rv = sphconv.RangeVoxel.from_sparse(x)
    assert tuple(rv.shape) == (B, C, D_, H_, W_)
    back = rv.to_sparse()
    assert torch.equal(back.z_idx, x.z_idx) and torch.equal(back.z_ptr, x.z_ptr)
    assert torch.equal(back.feature, x.feature)
    assert torch.equal(rv.dense(), x.dense().permute(0, 1, 4, 2, 3))
    with pytest.raises(AssertionError):
        sphconv.RangeVoxel(rv.feature, rv.depth, rv.thick, (B, C + 1, D_, H_, W_))


@pytest.mark.parametrize("subm,stride,padding", [(True, 1, 1), (False, 2, 1)])
def test_real_scan_through_the_whole_path(subm, stride, padding):
    """The reference's 'real' inputs (test/common.py:30-59: scan file -> voxels -> mean VFE, batch of
    two, channels repeated to 8; used at test_grad.py:192-299, 428-563): forward, dgrad and wgrad of one
    layer against torch's dense conv3d autograd in float64."""
    import os
    from sphconv_amd.datagen import VoxelizationVFE, merge_batch_torch
    kitti = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kitti_000000_reduced.bin")
    shape, B, ic, oc = [8, 32, 32], 2, 8, 16                       # spatial_shape_DWH
    vvfe = VoxelizationVFE(resolution_HWD=shape[::-1])
    voxels, coords = vvfe.generate(kitti, torch.device(G.DEV))
    ex = merge_batch_torch([{"voxels": voxels, "coordinates": coords}] * B)
    feat = ex["voxels"].repeat((1, 2))[:, :ic].contiguous()
    idx = ex["coordinates"].contiguous()
    assert idx.shape[0] > 1000
    cls = sphconv.SubMConv3d if subm else sphconv.SparseConv3d
    conv = cls(ic, oc, 3, stride=stride, padding=padding, bias=False).to(G.DEV)
    f = feat.clone().requires_grad_(True)
    x = sphconv.SparseConvTensor(f, shape, B, indices=idx)
    dense_y = conv(x).dense()
    w64 = conv.weight.detach().double().cpu().requires_grad_(True)
    f64 = feat.detach().double().cpu().requires_grad_(True)
    c = idx.long().cpu()
    d_in = torch.zeros((B, *shape, ic), dtype=torch.float64).index_put((c[:, 0], c[:, 1], c[:, 2], c[:, 3]), f64)
    ref = torch.nn.functional.conv3d(d_in.permute(0, 4, 1, 2, 3), w64.permute(4, 3, 0, 1, 2), None, stride, padding)
    if subm:
        mask = torch.zeros((B, 1, *shape), dtype=torch.float64)
        mask[c[:, 0], 0, c[:, 1], c[:, 2], c[:, 3]] = 1
        ref = ref * mask
    scale = float(ref.detach().abs().max())
    torch.testing.assert_close(dense_y.detach().double().cpu(), ref.detach(), rtol=1e-4, atol=1e-5 * scale)
    up = torch.randn(ref.shape, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    up = up * (mask if subm else (ref.detach().abs().sum(1, keepdim=True) != 0))
    (ref * up).sum().backward()
    (dense_y * up.to(G.DEV).float()).sum().backward()
    torch.testing.assert_close(f.grad.double().cpu(), f64.grad, rtol=1e-4, atol=1e-5 * float(f64.grad.abs().max()))
    torch.testing.assert_close(conv.weight.grad.double().cpu(), w64.grad, rtol=1e-4,
                               atol=1e-5 * float(w64.grad.abs().max()))


def test_scan_pipeline_matches_the_plain_path():
    """ScanPipeline (scans in flight on several HIP streams) returns what get_rulebook_subm + rule_conv return
    for every scan, whatever slot it lands in: the same bits with two launches per scan when the plain path takes
    the same kernels (books by groups), the same values to the path's tolerance otherwise (one launch, or a plain
    path that goes by rows: another order of summation)."""
    from sphconv_amd import sphconv_cuda as ext
    from sphconv_amd.pipeline import ScanPipeline
    from sphconv_amd.rulebook import RuleBook
    B, shape, ic, oc = 2, [10, 24, 16], 16, 32
    rng = np.random.default_rng(3)
    w = G.t((rng.standard_normal((3, 3, 3, ic, oc)) * 0.1).astype(np.float32)).half()
    for fused in (True, False):
        pipe = ScanPipeline(w, B, shape, max_voxels=4096, streams=3, fused=fused)
        assert pipe.streams == 3
        assert pipe.launches_for(4096) == (1 if fused else 2) and pipe.launches_for(128 * 769) == 2
        scans = []
        for s in range(7):                                     # more scans than slots, different sizes
            idx, feat = _inputs(10 + s, B, shape, ic, p=0.1 + 0.05 * s)
            x = sphconv.SparseConvTensor(G.t(feat).half(), shape, B, indices=G.t(idx))
            book = RuleBook.build_subm(x.z_idx, x.z_ptr, B, shape, [3, 3, 3])
            by_rows = book.fwd.tile_nbr is not None
            want = ext.rule_conv(x.feature, w.view(27, ic, oc), book, None, x.feature.shape[0])
            scans.append((x, want))
        torch.cuda.synchronize()

        def same(o, wnt):
            # two launches per scan: the very kernels of the plain path; one launch: the same pairs, added in another order
            if fused or by_rows:
                G.assert_same_conv(o, wnt)
            else:
                assert torch.equal(o, wnt)

        pending = []
        for i, (x, want) in enumerate(scans):
            out, slot = pipe.submit(x.feature, x.z_idx, x.z_ptr, row_cols=x.row_cols if i % 2 else None)
            pending.append((out, slot, want))
            if len(pending) == pipe.streams:                   # read a slot before it is used again
                o, sl, wnt = pending.pop(0)
                pipe.wait(sl)
                same(o, wnt)
        pipe.synchronize()
        for o, sl, wnt in pending:
            same(o, wnt)
    # a new weight is taken by the scans submitted after it
    pipe.set_weight(2 * w)
    out, slot = pipe.submit(scans[0][0].feature, scans[0][0].z_idx, scans[0][0].z_ptr)
    pipe.wait(slot)
    torch.testing.assert_close(out.float(), 2 * scans[0][1].float(), rtol=1e-2, atol=2e-3)
    with pytest.raises(sphconv.SphconvError):
        big = torch.zeros((5000, ic), dtype=torch.float16, device=G.DEV)
        pipe.submit(big, torch.zeros(5000, dtype=torch.int32, device=G.DEV), scans[0][0].z_ptr)


def test_fused_eval_tail_equals_separate_modules():
    """conv + BatchNorm1d(eval) + ReLU as one kernel against the same modules run one by one."""
    from sphconv_amd.synth import encoder_stack
    B, shape = 2, [16, 32, 16]
    idx, feat = _inputs(5, B, shape, 16)
    net = encoder_stack(16, (16, 32), seed=1).to(G.DEV).half()
    x = sphconv.SparseConvTensor(G.t(feat).half(), shape, B, indices=G.t(idx))
    with torch.no_grad():
        fused = net(x)
        net.fuse_eval = False
        x2 = sphconv.SparseConvTensor(G.t(feat).half(), shape, B, indices=G.t(idx))
        plain = net(x2)
    assert torch.equal(fused.z_idx, plain.z_idx) and torch.equal(fused.z_ptr, plain.z_ptr)
    assert float(plain.feature.float().abs().mean()) > 1e-2
    # the separate modules round to fp16 after the convolution and again after the batch norm
    torch.testing.assert_close(fused.feature.float(), plain.feature.float(), rtol=2e-2, atol=2e-2)
    # the affine map kept on a BatchNorm module follows in-place changes of its tensors
    net.fuse_eval = True
    with torch.no_grad():
        w0, m0 = net[1].weight.clone(), net[1].running_mean.clone()
        net[1].weight.mul_(-1.5)
        net[1].running_mean.add_(0.25)
        fused2 = net(sphconv.SparseConvTensor(G.t(feat).half(), shape, B, indices=G.t(idx)))
        net.fuse_eval = False
        plain2 = net(sphconv.SparseConvTensor(G.t(feat).half(), shape, B, indices=G.t(idx)))
        net[1].weight.copy_(w0)
        net[1].running_mean.copy_(m0)
    assert not torch.allclose(plain2.feature.float(), plain.feature.float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(fused2.feature.float(), plain2.feature.float(), rtol=3e-2, atol=5e-2)
    # with gradients enabled nothing is fused (autograd needs the separate modules)
    net.fuse_eval = True
    x3 = sphconv.SparseConvTensor(G.t(feat).half(), shape, B, indices=G.t(idx))
    y3 = net(x3)
    assert y3.feature.requires_grad
    assert torch.equal(y3.feature.detach(), plain.feature)


def test_strided_row_counts_started_ahead_change_nothing():
    """A container starts a strided layer's output-row count when the layer's input coordinates exist and
    hands it to the layer when it runs: same coordinates, same features, bit for bit, as counting where the
    layer runs -- under no_grad (fused tails) and with autograd; and the two halves used directly."""
    from sphconv_amd import _lib as L
    from sphconv_amd.rulebook import RuleBook
    from sphconv_amd.synth import encoder_stack
    B, shape = 3, [16, 40, 16]
    idx, feat = _inputs(9, B, shape, 16, p=0.15)
    net = encoder_stack(16, (16, 32, 32), seed=2).to(G.DEV).half()
    assert net.count_ahead
    outs = {}
    for ahead in (True, False):
        net.count_ahead = ahead
        with torch.no_grad():
            y = net(sphconv.SparseConvTensor(G.t(feat).half(), shape, B, indices=G.t(idx)))
        outs[ahead] = y
        f = G.t(feat).half().requires_grad_(True)
        yg = net(sphconv.SparseConvTensor(f, shape, B, indices=G.t(idx)))
        yg.feature.float().square().sum().backward()
        outs[ahead, "grad"] = (yg.feature.detach(), f.grad.clone(), [p.grad.clone() for p in net.parameters() if p.grad is not None])
        net.zero_grad()
    net.count_ahead = True
    a, b = outs[True], outs[False]
    assert a.feature.shape[0] > 0 and float(a.feature.float().abs().mean()) > 1e-3
    assert torch.equal(a.z_idx, b.z_idx) and torch.equal(a.z_ptr, b.z_ptr) and torch.equal(a.feature, b.feature)
    (ya, ga, pa), (yb, gb, pb) = outs[True, "grad"], outs[False, "grad"]
    assert torch.equal(ya, yb) and torch.equal(ga, gb) and len(pa) == len(pb) > 0
    assert all(torch.equal(u, v) for u, v in zip(pa, pb))
    # the two halves by hand, with other work (another strided layer's rules) enqueued in between
    x = sphconv.SparseConvTensor(G.t(feat).half(), shape, B, indices=G.t(idx))
    args = (x.z_idx, x.z_ptr, B, shape, [8, 20, 8], [3, 3, 3], [2, 2, 2], [1, 1, 1])
    h = RuleBook.count_ahead(*args)
    other = RuleBook.build(x.z_idx, x.z_ptr, B, shape, [14, 38, 14], [3, 3, 3], [1, 1, 1], [0, 0, 0])
    late = RuleBook.build(*args, ahead=h)
    plain = RuleBook.build(*args)
    assert other.out_rows > 0 and late.out_rows == plain.out_rows > 0
    assert torch.equal(late.oz_idx, plain.oz_idx) and torch.equal(late.oz_ptr, plain.oz_ptr)
    assert np.array_equal(G.book_triples(late.fwd), G.book_triples(plain.fwd))
    # a count started for one layer is refused by another
    h2 = RuleBook.count_ahead(*args)
    with pytest.raises(L.SphconvError, match="another layer"):
        RuleBook.build(x.z_idx, x.z_ptr, B, shape, [14, 38, 14], [3, 3, 3], [1, 1, 1], [0, 0, 0], ahead=h2)


def test_config4_encoder_full_size_layer_by_layer():
    """BASELINE configuration 4 (batch 4, grid 64x2048x64, four stages of two submanifold and one
    strided convolution, BatchNorm + ReLU fused, fp16): every layer's output against the C oracle
    applied to that layer's own input, rules included."""
    from sphconv_amd.synth import encoder_stack
    d = make_config(4, seed=0)
    shape, B = d["spatial_shape"], d["batch"]
    n = d["z_idx"].shape[0]
    rng = np.random.default_rng(4)
    feat = torch.tensor(rng.standard_normal((n, 16)), dtype=torch.float32).half()
    net = encoder_stack(16, (16, 32, 64, 64), seed=4).to(G.DEV).half()
    x = sphconv.SparseConvTensor(feat.to(G.DEV), shape, B, z_idx=G.t(d["z_idx"]), z_ptr=G.t(d["z_ptr"]))
    mods = list(net)
    with torch.no_grad():
        for i in range(0, len(mods), 3):
            conv, bn = mods[i], mods[i + 1]
            z_idx, z_ptr = x.z_idx.cpu().numpy(), x.z_ptr.cpu().numpy()
            f_in = x.feature.float().cpu().numpy()
            in_shape = [x.D, x.W, x.H]
            y = sphconv.Sequential(*mods[i:i + 3])(x)
            if conv.subm:
                oshape = in_shape
                ora = O.get_rules_subm(z_idx, z_ptr, B, in_shape, oshape, [3, 3, 3], [1, 1, 1], [1, 1, 1], n_max=512)
            else:
                oshape = H.out_shape_of(in_shape, [3, 3, 3], [2, 2, 2], [1, 1, 1])
                ora = O.get_rules(z_idx, z_ptr, B, in_shape, oshape, [3, 3, 3], [2, 2, 2], [1, 1, 1], n_max=512)
            oz_idx, oz_ptr, rules, rule_size, dropped = ora
            assert dropped == 0
            assert [y.D, y.W, y.H] == list(oshape)
            assert np.array_equal(y.z_idx.cpu().numpy(), oz_idx) and np.array_equal(y.z_ptr.cpu().numpy(), oz_ptr)
            w = conv.weight.detach().float().cpu().numpy().reshape(27, conv.in_channels, conv.out_channels)
            acc = O.rule_conv(f_in, w, rules, rule_size, oz_idx.shape[0])
            scale = (bn.weight.float() / torch.sqrt(bn.running_var.float() + bn.eps)).cpu().numpy()
            shift = (bn.bias.float() - bn.running_mean.float() * bn.weight.float()
                     / torch.sqrt(bn.running_var.float() + bn.eps)).cpu().numpy()
            want = np.maximum(acc * scale[None, :] + shift[None, :], 0.0)
            got = y.feature.float().cpu().numpy()
            assert got.shape == want.shape
            # fp32 accumulate, one rounding to fp16 (tolerance of the task: rtol 1e-2, atol 1e-3)
            assert (np.abs(got - want) <= 2.0 ** -9 * np.abs(want) + 1e-3).all(), i
            assert 0.2 < (want > 0).mean() < 0.9 and 1e-2 < np.abs(want).mean() < 1e2, (i, np.abs(want).mean())
            x = y
    assert [x.D, x.W, x.H] == [4, 128, 4] and x.feature.shape[1] == 64


def test_packed_weight_is_kept_only_on_request_and_follows_updates():
    """The fragment-ordered copy of a weight is made on every call unless the caller asks to keep it (modules do
    in eval mode under torch.no_grad()); a kept copy is reused until the weight's version counter moves (an
    in-place update).  Updates through `.data` do not move the counter: they are seen at once by a module in
    training mode, and by one in eval mode after `invalidate_packed()`."""
    from sphconv_amd import sphconv_cuda as ext
    B, shape = 1, [8, 16, 8]
    idx, feat = _inputs(3, B, shape, 16)
    conv = sphconv.SubMConv3d(16, 32, 3).to(G.DEV).half()
    x = sphconv.SparseConvTensor(G.t(feat).half(), shape, B, indices=G.t(idx))
    w = conv.weight.view(-1, 16, 32)
    with torch.no_grad():
        assert ext._packed_weight(w, False) is not ext._packed_weight(w, False)     # not asked to keep: a copy per call
        p1 = ext._packed_weight(w, False, cache=True)
        assert ext._packed_weight(conv.weight.view(-1, 16, 32), False, cache=True) is p1   # another view of the parameter
        assert ext._packed_weight(w, True, cache=True) is not p1                      # other form, other copy
        conv.eval()
        y1 = conv(x).feature.clone()
        conv.weight.mul_(2.0)                                                         # bumps the version counter
        p2 = ext._packed_weight(w, False, cache=True)
        assert p2 is not p1 and not torch.equal(p2, p1)
        y2 = conv(x).feature.clone()
        torch.testing.assert_close(y2.float(), 2 * y1.float(), rtol=2e-3, atol=2e-3)
        # through .data the version counter stays: eval mode keeps the old copy until it is told
        v = conv.weight._version
        conv.weight.data.mul_(2.0)
        assert conv.weight._version == v
        conv.invalidate_packed()
        y3 = conv(x).feature.clone()
        torch.testing.assert_close(y3.float(), 4 * y1.float(), rtol=2e-3, atol=4e-3)
        # a module in training mode keeps nothing: the same kind of update is seen without being told
        conv.train()
        conv.weight.data.mul_(0.5)
        y4 = conv(x).feature
        torch.testing.assert_close(y4.float(), 2 * y1.float(), rtol=2e-3, atol=2e-3)
    with torch.enable_grad():
        assert ext._packed_weight(w, False, cache=True) is not ext._packed_weight(w, False, cache=True)
