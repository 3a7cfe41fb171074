"""CPU-only checks of the host side: the C-ABI library loads and exports every
symbol the public header declares, host arithmetic, and error paths that need no
GPU.  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

import sphconv_amd
from oracle import oracle as O
from sphconv_amd import _lib as L
from sphconv_amd import utils

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "sphconv_hip.h")).read()
    declared = set(re.findall(r"\b(sph_[a-z0-9_]+)\s*\(", hdr))
    declared -= {"sph_status", "sph_dtype"}
    assert declared, "no declarations found"
    assert os.path.exists(L.LIB_PATH), "libsphconv_hip.so is not built"
    lib = ctypes.CDLL(L.LIB_PATH)
    missing = [s for s in sorted(declared) if not hasattr(lib, s)]
    assert not missing, missing
    assert declared == set(L.EXPORTS), declared ^ set(L.EXPORTS)


def test_host_arithmetic_matches_oracle_closed_forms():
    lib = L.lib()
    assert lib.sph_abi_version() == L.ABI_VERSION
    assert lib.sph_book_tiles(0) == 0 and lib.sph_book_tiles(1) == 1 and lib.sph_book_tiles(129) == 2
    assert lib.sph_book_cap(27) == 27 * 8
    for B, shape, K, s, T, nnz in [(1, [64, 512, 32], [3, 3, 3], [1, 1, 1], [2, 2], 39256),
                                   (4, [64, 2048, 64], [3, 3, 3], [2, 2, 2], [2, 2], 630544),
                                   (8, [64, 512, 32], [3, 3, 3], [1, 1, 1], [4, 8], 314214),
                                   (2, [7, 9, 11], [2, 3, 1], [1, 2, 1], [3, 1], 50)]:
        out = utils.out_spatial(shape, K, s, [1, 1, 1])
        g = L.make_geom(B, shape, out, K, s, [1, 1, 1])
        assert lib.sph_tile_n_max(ctypes.byref(g), T[0], T[1], nnz) == O.tile_n_max(B, shape, K, s, T, nnz)
        assert lib.sph_num_tiles(ctypes.byref(g), T[0], T[1]) == -(-out[0] // T[0]) * -(-out[1] // T[1])
        assert out == O.out_spatial(shape, K, s, [1, 1, 1])


def test_argument_errors_without_gpu():
    lib = L.lib()
    g = L.make_geom(1, [4, 4, 4], [4, 4, 4], [7, 7, 7], [1, 1, 1], [3, 3, 3])     # KV = 343 > 128
    assert lib.sph_outcoords_blocks(ctypes.byref(g)) < 0
    assert b"geometry" in lib.sph_last_error()
    assert lib.sph_weight_packed_bytes(L.F16, 27, 64, 64) == 27 * 2 * 4 * 64 * 16
    assert lib.sph_weight_packed_bytes(L.F32, 27, 16, 16) == 27 * 1 * 1 * 64 * 16
    assert lib.sph_weight_packed_bytes(7, 27, 16, 16) == 0
    rc = lib.sph_conv_apply(L.F16, None, 0, 64, None, 64, None, None, None, None)
    assert rc == -1 and b"book" in lib.sph_last_error()
    with pytest.raises(L.SphconvError):
        L.check(rc)
    with pytest.raises(L.SphconvError):
        L.dtype_code(torch.float64)
    with pytest.raises(L.SphconvError):
        L.ptr(torch.zeros(4))            # not a GPU tensor


def test_module_construction_and_init():
    conv = sphconv_amd.SubMConv3d(16, 32, 3, padding=0, indice_key="k")
    assert tuple(conv.weight.shape) == (3, 3, 3, 16, 32) and conv.padding == (1, 1, 1) and conv.subm
    assert conv.bias is None and conv.rule_size is None
    # fan_in = oC * KV (reference utils/__init__.py:69-75): bound = sqrt(6/((1+5)*fan_in))
    bound = (6.0 / (6.0 * 32 * 27)) ** 0.5
    assert conv.weight.abs().max().item() <= bound
    c2 = sphconv_amd.SparseConv3d(4, 8, [3, 1, 3], stride=[2, 1, 2], padding=[1, 0, 1], bias=True)
    assert tuple(c2.weight.shape) == (3, 1, 3, 4, 8) and c2.bias.shape == (8,)
    assert "stride=(2, 1, 2)" in repr(c2)
    seq = sphconv_amd.SparseSequential(conv, torch.nn.ReLU(), c=c2)
    assert len(seq) == 3 and seq[0] is conv and seq[-1] is c2
    assert utils.out_spatial([64, 2048, 64], [3, 3, 3], [2, 2, 2], [1, 1, 1]) == [32, 1024, 32]
    assert utils._triple(3) == (3, 3, 3) and utils._triple([1, 2, 3]) == (1, 2, 3)
    sd = conv.state_dict()
    assert list(sd) == ["weight"]


def test_bench_refuses_more_than_one_gpu():
    """The path runs on one GPU; bench.py says so and exits before touching any device."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout == ""


def test_training_channel_limit_is_reported_before_forward():
    """Forward takes up to 256 input channels, dgrad/wgrad up to 128: a module that wants gradients says so
    when it is called, not from inside backward()."""
    import torch
    import sphconv_amd
    from sphconv_amd.functional import ConvFunction
    feature = torch.zeros((4, 192), requires_grad=True)
    weight = torch.zeros((27, 192, 32), requires_grad=True)
    with pytest.raises(sphconv_amd.SphconvError, match="training takes 1..128 input channels"):
        ConvFunction.apply(feature, weight, None, None, [1, 1], 4)
