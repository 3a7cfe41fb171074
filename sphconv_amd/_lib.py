"""ctypes binding of ``libsphconv_hip.so`` (the C ABI declared in
``include/sphconv_hip.h``).  PyTorch is used only to own device memory and the
current HIP stream; every computation on the path happens inside the library.

There is no CPU fallback: if the library is missing or a call fails, an
exception is raised.
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsphconv_hip.so")

TILE_ROWS = 128
GROUP = 16
STATIC_MAX_COLUMNS = 1 << 20     # SPH_STATIC_MAX_COLUMNS of the header

F32, F16, BF16, I8 = 0, 1, 2, 3
ERR_ARG, ERR_UNSUPPORTED, ERR_LAUNCH = -1, -2, -3      # sph_status
FUSED_WRITE_BOOK, FUSED_IN_FLIGHT = 1, 2               # flags of sph_rules_conv
_DTYPES = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.int8: I8}


class SphconvError(RuntimeError):
    pass


class Geom(C.Structure):
    _fields_ = [("B", C.c_int32), ("S", C.c_int32 * 3), ("O", C.c_int32 * 3),
                ("K", C.c_int32 * 3), ("stride", C.c_int32 * 3), ("pad", C.c_int32 * 3),
                ("dil", C.c_int32 * 3)]


class Book(C.Structure):
    _fields_ = [("tile_ngrp", C.c_void_p), ("tile_koff", C.c_void_p), ("grp_k", C.c_void_p),
                ("grp_gather", C.c_void_p), ("grp_owner", C.c_void_p), ("rows", C.c_int32),
                ("KV", C.c_int32), ("tile_nbr", C.c_void_p), ("middle_run", C.c_int32)]


class Epilogue(C.Structure):
    _fields_ = [("scale", C.c_void_p), ("shift", C.c_void_p), ("relu", C.c_int32)]


_lib = None
ABI_VERSION = 7       # sph_abi_version() of the library these signatures describe

_I, _P, _L, _Z = C.c_int, C.c_void_p, C.c_long, C.c_size_t
_SIGNATURES = {
    "sph_last_error": (C.c_char_p, []),
    "sph_abi_version": (_I, []),
    "sph_book_tiles": (_I, [_I]),
    "sph_book_cap": (_I, [_I]),
    "sph_tile_n_max": (_I, [C.POINTER(Geom), _I, _I, _I]),
    "sph_num_tiles": (_I, [C.POINTER(Geom), _I, _I]),
    "sph_rules_build": (_I, [_P, _P, _I, _P, _P, _I, C.POINTER(Geom), _I, C.POINTER(Book), _P, _P]),
    "sph_rules_build_pack": (_I, [_P, _P, _I, _P, _P, _I, C.POINTER(Geom), _I, C.POINTER(Book), _P, _I, _P, _I, _I, _I, _L,
                                  _L, _L, _P, _P]),
    "sph_row_columns": (_I, [_P, _I, _I, _P, _P]),
    "sph_outcoords_blocks": (_I, [C.POINTER(Geom)]),
    "sph_outcoords_scratch_ints": (_I, [C.POINTER(Geom)]),
    "sph_outcoords_state_ints": (_I, [C.POINTER(Geom)]),
    "sph_outcoords_count": (_I, [_P, _P, _I, C.POINTER(Geom), _P, _P, _P, _P]),
    "sph_outcoords_count_static": (_I, [_P, _P, _I, C.POINTER(Geom), _P, _P, C.POINTER(C.c_void_p), _P]),
    "sph_outcoords_fill": (_I, [_P, _P, _I, C.POINTER(Geom), _P, _P, _P, _I, _P, _P]),
    "sph_rules_to_padded_count": (_I, [C.POINTER(Book), _P, C.POINTER(Geom), _I, _I, _P, _P, _P]),
    "sph_rules_to_padded_fill": (_I, [_P, C.POINTER(Geom), _I, _I, _P, _I, _I, _I, _P, _P]),
    "sph_rules_from_padded": (_I, [_P, _P, _I, _I, _I, _I, _I, _I, _P, C.POINTER(Book), _P]),
    "sph_weight_packed_bytes": (_Z, [_I, _I, _I, _I]),
    "sph_weight_pack": (_I, [_I, _P, _I, _I, _I, _L, _L, _L, _P, _P]),
    "sph_conv_apply": (_I, [_I, _P, _I, _I, _P, _I, C.POINTER(Book), C.POINTER(Epilogue), _P, _P]),
    "sph_rules_conv": (_I, [_P, _P, _I, _P, _P, _I, C.POINTER(Geom), C.POINTER(Book), _I, _P, _I, _P, _I, _P, _I,
                            C.POINTER(Epilogue), _P, _P]),
    "sph_wgrad_partial_elems": (_Z, [_I, _I, _I, _I]),
    "sph_conv_wgrad": (_I, [_I, _P, _I, _I, _P, _I, C.POINTER(Book), _P, _P, _I, _P]),
    "sph_init_tensor_workspace": (_Z, [_I, _I, _I, _I, _I]),
    "sph_init_tensor": (_I, [_P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _Z, _P]),
    "sph_permute_rows": (_I, [_P, _P, _I, _I, _I, _P, _P]),
    "sph_points_to_voxel_workspace": (_Z, [_I, _I, _I, _I]),
    "sph_points_to_voxel": (_I, [_P, _I, _I, _I, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float, _I, _I,
                                 _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "sph_xyz_to_rangevoxel": (_I, [_P, _I, _I, _I, _I, _I, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float,
                                   C.c_float, _I, _P, _P, _P, _P, _P, _P]),
    "sph_to_dense": (_I, [_P, _P, _P, _I, _I, _I, _I, _P, _P]),
    "sph_to_dense_backward": (_I, [_P, _P, _P, _I, _I, _I, _I, _P, _P]),
}
EXPORTS = tuple(_SIGNATURES)


def lib():
    """The loaded library; raises SphconvError if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SphconvError(
                "libsphconv_hip.so is not built (run `make -C sphconv_amd/csrc` or "
                "`python -c 'import __graft_entry__ as g; g.build()'`); there is no CPU fallback")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        if handle.sph_abi_version() != ABI_VERSION:
            raise SphconvError("%s has ABI version %d, this package needs %d: rebuild it (make -C sphconv_amd/csrc)"
                               % (LIB_PATH, handle.sph_abi_version(), ABI_VERSION))
        _lib = handle
    return _lib


def check(rc: int):
    if rc != 0:
        raise SphconvError("libsphconv_hip: %s (status %d)" % (lib().sph_last_error().decode(), rc))


def dtype_code(t: torch.dtype) -> int:
    try:
        return _DTYPES[t]
    except KeyError:
        raise SphconvError("unsupported element type %s (float32, float16, bfloat16, int8)" % t)


def ptr(t):
    """Device pointer of a contiguous CUDA tensor (None -> NULL)."""
    if t is None:
        return None
    if not t.is_cuda:
        raise SphconvError("expected a GPU tensor, got device %s" % t.device)
    if not t.is_contiguous():
        raise SphconvError("expected a contiguous tensor")
    return t.data_ptr()


def stream():
    """Raw handle of torch's current HIP stream on the current device."""
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())


def make_geom(batch, in_shape, out_shape, kernel, stride, padding, dilation=(1, 1, 1)) -> Geom:
    g = Geom()
    g.B = int(batch)
    for d in range(3):
        g.S[d] = int(in_shape[d])
        g.O[d] = int(out_shape[d])
        g.K[d] = int(kernel[d])
        g.stride[d] = int(stride[d])
        g.pad[d] = int(padding[d])
        g.dil[d] = int(dilation[d])
    return g
