"""sph_outcoords_count_static: the output-coordinate count + scan for callers that cannot allocate
(its scratch is an array of the library's own) against sph_outcoords_count with a scratch of the
caller's, through the C ABI: bit-exact oz_ptr, row count and (through sph_outcoords_fill on the
scratch pointer it returns) oz_idx, on two calls in a row, the second on a smaller input."""
import ctypes as C

import numpy as np
import pytest
import torch

import helpers as H
import gpu_helpers as G
from sphconv_amd import _lib as L

pytestmark = pytest.mark.gpu


def _case(seed, B, shape, p):
    rng = np.random.default_rng(seed)
    idx = np.argwhere(rng.random((B, *shape)) < p).astype(np.int32)
    _, z_idx, z_ptr, _ = H.csr_from_indices(idx, B, shape)
    return G.t(z_idx), G.t(z_ptr), H.out_shape_of(shape, [3, 3, 3], [2, 2, 2], [1, 1, 1])


def _run(lib, zi, zp, B, shape, out_shape, static):
    g = L.make_geom(B, shape, out_shape, [3, 3, 3], [2, 2, 2], [1, 1, 1], [1, 1, 1])
    n_in = int(zi.shape[0])
    oz_ptr = torch.full((B, out_shape[0], out_shape[1]), -1, dtype=torch.int32, device=G.DEV)
    total = torch.full((1,), -1, dtype=torch.int32, device=G.DEV)
    if static:
        sp = C.c_void_p()
        L.check(lib.sph_outcoords_count_static(L.ptr(zi), L.ptr(zp), n_in, C.byref(g), L.ptr(oz_ptr), L.ptr(total),
                                               C.byref(sp), L.stream()))
        scratch_ptr = sp.value
        assert scratch_ptr
    else:
        n = lib.sph_outcoords_scratch_ints(C.byref(g))
        scratch = torch.zeros(n + (n & 1), dtype=torch.int32, device=G.DEV)
        L.check(lib.sph_outcoords_count(L.ptr(zi), L.ptr(zp), n_in, C.byref(g), L.ptr(oz_ptr), L.ptr(scratch),
                                        L.ptr(total), L.stream()))
        scratch_ptr = scratch.data_ptr()
    m = int(total.item())
    oz_idx = torch.full((max(m, 1),), -1, dtype=torch.int32, device=G.DEV)
    L.check(lib.sph_outcoords_fill(L.ptr(zi), L.ptr(zp), n_in, C.byref(g), scratch_ptr, L.ptr(oz_ptr), L.ptr(oz_idx), m,
                                   None, L.stream()))
    torch.cuda.synchronize()
    return oz_ptr.cpu().numpy(), m, oz_idx.cpu().numpy()


def test_static_scratch_matches_caller_scratch_twice():
    lib = L.lib()
    # first a grid of hundreds of scan workgroups, then a much smaller one: the array keeps the first call's contents
    # (and last one whose columns keep three masks each: 150 bins)
    for seed, B, shape, p in ((1, 4, [64, 512, 32], 0.05), (2, 1, [9, 33, 12], 0.3), (3, 2, [16, 40, 300], 0.05)):
        zi, zp, out_shape = _case(seed, B, shape, p)
        got = _run(lib, zi, zp, B, shape, out_shape, static=True)
        want = _run(lib, zi, zp, B, shape, out_shape, static=False)
        assert got[1] == want[1] and got[1] > 0
        assert np.array_equal(got[0], want[0])
        assert np.array_equal(got[2], want[2])
        assert (got[2][:got[1]] >= 0).all()


def test_static_scratch_allocates_nothing_and_is_one_array():
    """What the entry point is for: between two calls the device's free memory does not move (no allocation, no
    free, in the library or through torch), and every call names the same array."""
    lib = L.lib()
    zi, zp, out_shape = _case(4, 2, [32, 96, 24], 0.1)
    B, shape = 2, [32, 96, 24]
    g = L.make_geom(B, shape, out_shape, [3, 3, 3], [2, 2, 2], [1, 1, 1], [1, 1, 1])
    oz_ptr = torch.empty((B, out_shape[0], out_shape[1]), dtype=torch.int32, device=G.DEV)
    total = torch.empty((1,), dtype=torch.int32, device=G.DEV)
    ptrs = []

    def call():
        sp = C.c_void_p()
        L.check(lib.sph_outcoords_count_static(L.ptr(zi), L.ptr(zp), int(zi.shape[0]), C.byref(g), L.ptr(oz_ptr),
                                               L.ptr(total), C.byref(sp), L.stream()))
        ptrs.append(sp.value)

    call()                                  # the first call on a device looks the array's address up
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0 = torch.cuda.memory_reserved()
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0 and torch.cuda.memory_reserved() == reserved0
    assert len(set(ptrs)) == 1 and ptrs[0]
    assert int(total.item()) > 0


def test_static_scratch_rejects_grids_beyond_its_size():
    lib = L.lib()
    limit = L.STATIC_MAX_COLUMNS
    B, shape = 1, [2048, 2 * (limit // 2048) + 2, 4]       # more output columns than the array provides for
    out_shape = shape
    g = L.make_geom(B, shape, out_shape, [3, 3, 3], [1, 1, 1], [1, 1, 1], [1, 1, 1])
    assert B * out_shape[0] * out_shape[1] > limit
    zi = torch.zeros(1, dtype=torch.int32, device=G.DEV)
    zp = torch.zeros(8, dtype=torch.int32, device=G.DEV)       # never read: the call is refused before any launch
    sp = C.c_void_p()
    rc = lib.sph_outcoords_count_static(L.ptr(zi), L.ptr(zp), 0, C.byref(g), L.ptr(zp), None, C.byref(sp), L.stream())
    assert rc == -2 and b"scratch provides for" in lib.sph_last_error()
