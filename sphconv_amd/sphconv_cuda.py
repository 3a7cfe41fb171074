"""The reference's extension module, re-implemented over ``libsphconv_hip.so``.

Same function names, argument order and return values as the pybind11 module
``sphconv.sphconv_cuda`` (src/sphconv/all.cpp:18-31), so code written against the
reference (``from sphconv.sphconv_cuda import get_rules, rule_conv ...``) runs
unchanged with ``sphconv_amd.sphconv_cuda``.  Differences, all additive:

* fibers come out of ``init_tensor`` sorted by S2 and rule lists sorted by row
  (the reference leaves both in atomic-race order);
* ``rules`` may be a :class:`~sphconv_amd.rulebook.RuleBook` (what
  :func:`get_rulebook` / :func:`get_rulebook_subm` return) wherever the reference
  takes its padded tensor -- the fast path that never materialises the padding;
* float16 / bfloat16 features (fp32 accumulate) and int8 (:func:`rule_conv_int8`);
* bad arguments raise ``SphconvError`` / ``ValueError`` instead of aborting.
"""
import ctypes as C
import weakref
from typing import List, Optional, Sequence

import torch

from . import _lib as L
from .rulebook import RuleBook

# channel limits of the kernels: forward contracts over up to 256 input channels into up to 128 output
# channels; dgrad writes iC columns and wgrad keeps an iC x oC tile per offset, so training needs both <= 128
MAX_FORWARD_IN_CHANNELS = 256
MAX_OUT_CHANNELS = 128
MAX_TRAIN_CHANNELS = 128

__version__ = "hip-gfx950"

# Packed copies of weights, kept only for callers that ask for it (``cache=True``: modules in eval mode, under
# ``torch.no_grad()``): one per (weight tensor, form), valid while the tensor object lives and its version
# counter, storage address, shape and type have not moved.
_PACKED_CACHE = {}


def invalidate_packed(weight: Optional[torch.Tensor] = None):
    """Forgets the kept packed copies of ``weight`` (all of them when None).  Needed after an update the version
    counter does not see: ``weight.data.mul_(2)`` or ``weight.data.copy_(...)`` change the values and leave
    ``weight._version`` where it was."""
    if weight is None:
        _PACKED_CACHE.clear()
        return
    base = weight._base if weight._base is not None else weight
    for key in [k for k in _PACKED_CACHE if k[0] == id(base)]:
        _PACKED_CACHE.pop(key, None)


def _packed_weight(weight: torch.Tensor, transpose: bool, reverse: bool = False, cache: bool = False) -> torch.Tensor:
    """weight [KV, a, b] -> fragment-ordered copy for the contraction over ``a``
    (``transpose``: over ``b``, i.e. with W[k]^T; ``reverse``: offsets in reverse order, W[KV-1-k]).
    The copy is made on every call (a weight may have been updated in place) unless the caller passes
    ``cache=True`` while no gradient is being recorded: then it is kept with the weight and reused until the
    weight's version counter, address, shape or type change.  Updates through ``weight.data`` do not move the
    version counter: call :func:`invalidate_packed` after them (modules: ``Convolution.invalidate_packed()``).
    The kept copy belongs to the stream it was made on; other streams must order themselves behind it."""
    w = weight.detach()
    if not w.is_contiguous():
        w = w.contiguous()
    cache_key = None
    if cache and not torch.is_grad_enabled() and w.data_ptr() == weight.data_ptr():
        base = weight._base if weight._base is not None else weight
        cache_key = (id(base), bool(transpose), bool(reverse), L.stream())
        state = (base._version, w.data_ptr(), tuple(w.shape), w.dtype)
        hit = _PACKED_CACHE.get(cache_key)
        if hit is not None and hit[0]() is base and hit[1] == state:
            return hit[2]
    lib = L.lib()
    kv, a, b = w.shape
    kdim, ndim = (b, a) if transpose else (a, b)
    skk, sn = (1, b) if transpose else (b, 1)
    dt = L.dtype_code(w.dtype)
    nbytes = lib.sph_weight_packed_bytes(dt, kv, kdim, ndim)
    if nbytes == 0:
        raise L.SphconvError("cannot pack weight of shape %s" % (tuple(w.shape),))
    packed = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    first, sk = L.ptr(w), a * b
    if reverse:                                  # start at the last offset and walk backwards
        first, sk = first + (kv - 1) * a * b * w.element_size(), -a * b
    L.check(lib.sph_weight_pack(dt, first, kv, kdim, ndim, sk, skk, sn, L.ptr(packed), L.stream()))
    if cache_key is not None:
        _PACKED_CACHE[cache_key] = (weakref.ref(base, lambda _r, k=cache_key: _PACKED_CACHE.pop(k, None)), state, packed)
    return packed


def _dgrad_buffers(book: RuleBook, d_out: torch.Tensor, kdim: int, ndim: int):
    """(buffers, reverse) for d_feature = sum d_out[out] @ W[k]^T.  A submanifold book with odd kernels is
    its own transpose with the offsets mirrored (the pair (k, in=i, out=j) has the twin (KV-1-k, in=j,
    out=i)): the forward book serves, with the weight's offsets reversed, and no transposed book is built."""
    if book.mirrored():
        fake_w = torch.empty((book.kv, kdim, ndim), dtype=d_out.dtype, device="meta")
        return _conv_buffers(book, d_out, fake_w, False), True
    return None, False


def _as_book(rules, rule_size, in_rows: int, out_rows: int) -> RuleBook:
    if isinstance(rules, RuleBook):
        return rules
    return RuleBook.from_padded(rules, rule_size, in_rows, out_rows)


_NO_EPILOGUE = L.Epilogue(None, None, 0)


def _apply(feature, packed, kdim, ndim, buffers, scale=None, shift=None, relu=False, out_dtype=None):
    if not feature.is_contiguous():
        feature = feature.contiguous()
    if not feature.is_cuda:
        raise L.SphconvError("expected a GPU tensor, got device %s" % feature.device)
    out = torch.empty((buffers.rows, ndim), dtype=out_dtype or feature.dtype, device=feature.device)
    if scale is None and shift is None and not relu:
        epi = _NO_EPILOGUE
    else:
        epi = L.Epilogue(L.ptr(scale), L.ptr(shift), int(bool(relu)))
    rc = L.lib().sph_conv_apply(L.dtype_code(feature.dtype), feature.data_ptr(), feature.shape[0], kdim,
                                packed.data_ptr(), ndim, C.byref(buffers.struct()), C.byref(epi),
                                out.data_ptr(), L.stream())
    if rc:
        L.check(rc)
    return out


# ---- tensor.h ---------------------------------------------------------------

def init_tensor(feature: torch.Tensor, indicesBZYX: torch.Tensor, batchSize: int,
                spatialShape: Sequence[int]) -> List[torch.Tensor]:
    """tensor.cu:78-127 -> [outFeature, zIndices, zPtr, permutation].  Rows of a
    fiber are ordered by ascending S2 (one legal order of the reference's output).
    One 8-byte device->host read checks the coordinates (the reference checks nothing:
    coordinates outside the grid or duplicated ones corrupt its output)."""
    if indicesBZYX.dtype != torch.int32 or indicesBZYX.dim() != 2 or indicesBZYX.shape[1] != 4:
        raise ValueError("indices must be int32 [NNZ,4] (b,s0,s1,s2)")
    if feature.dim() != 2 or feature.shape[0] != indicesBZYX.shape[0]:
        raise ValueError("feature must be [NNZ,C]")
    S0, S1, S2 = (int(v) for v in spatialShape)
    B = int(batchSize)
    n = feature.shape[0]
    dev = feature.device
    lib = L.lib()
    idx = indicesBZYX.contiguous()
    z_idx = torch.empty(n, dtype=torch.int32, device=dev)
    z_ptr = torch.empty((B, S0, S1), dtype=torch.int32, device=dev)
    permutation = torch.empty(n, dtype=torch.int32, device=dev)
    status = torch.empty(2, dtype=torch.int32, device=dev)
    nbytes = lib.sph_init_tensor_workspace(n, B, S0, S1, S2)
    if nbytes == 0:
        raise L.SphconvError("bad batch size / spatial shape %s" % ([B, S0, S1, S2],))
    work = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    L.check(lib.sph_init_tensor(L.ptr(idx), n, B, S0, S1, S2, L.ptr(z_idx), L.ptr(z_ptr), L.ptr(permutation),
                                L.ptr(status), L.ptr(work), nbytes, L.stream()))
    outside, dup = (int(v) for v in status.tolist())
    if outside:
        raise ValueError("voxel coordinate outside batch/spatial shape %s" % ([B, S0, S1, S2],))
    if dup:
        raise ValueError("duplicate voxel coordinates")
    feature = feature.contiguous()
    out = torch.empty_like(feature)
    L.check(lib.sph_permute_rows(L.ptr(feature), L.ptr(permutation), n,
                                 feature.shape[1] * feature.element_size(), 0, L.ptr(out), L.stream()))
    return [out, z_idx, z_ptr, permutation]


def init_tensor_backward(d_featureOut: torch.Tensor, permutation: torch.Tensor) -> torch.Tensor:
    """tensor.cu:147-162: d_feature[n] = d_featureOut[permutation[n]]."""
    d = d_featureOut.contiguous()
    out = torch.empty_like(d)
    L.check(L.lib().sph_permute_rows(L.ptr(d), L.ptr(permutation.contiguous()), d.shape[0],
                                     d.shape[1] * d.element_size(), 1, L.ptr(out), L.stream()))
    return out


def to_dense(feature: torch.Tensor, zIndices: torch.Tensor, zPtr: torch.Tensor, D: int,
             out: torch.Tensor) -> torch.Tensor:
    """tensor.cu:222-264: writes active cells of ``out`` [B,S0,S1,S2,C] and returns it."""
    feature = feature.contiguous()
    if out.dim() != 5 or out.shape[4] != feature.shape[1] or out.dtype != feature.dtype:
        raise ValueError("out must be [B,S0,S1,S2,C] of the feature's dtype")
    ncol = zPtr.numel()
    if out.shape[0] * out.shape[1] * out.shape[2] != ncol or out.shape[3] != int(D):
        raise ValueError("out shape %s does not match z_ptr %s and D=%d"
                         % (tuple(out.shape), tuple(zPtr.shape), D))
    L.check(L.lib().sph_to_dense(L.ptr(feature), L.ptr(zIndices), L.ptr(zPtr), feature.shape[0], ncol,
                                 int(D), feature.shape[1] * feature.element_size(), L.ptr(out), L.stream()))
    return out


def to_dense_backward(d_featureOut: torch.Tensor, zIndices: torch.Tensor, zPtr: torch.Tensor) -> torch.Tensor:
    """tensor.cu:266-309: gathers [B,S0,S1,S2,C] gradients at the active cells."""
    d = d_featureOut.contiguous()
    n, c = zIndices.shape[0], d.shape[4]
    out = torch.zeros((n, c), dtype=d.dtype, device=d.device)
    L.check(L.lib().sph_to_dense_backward(L.ptr(d), L.ptr(zIndices), L.ptr(zPtr), n, zPtr.numel(),
                                          d.shape[3], c * d.element_size(), L.ptr(out), L.stream()))
    return out


# ---- rules.h ----------------------------------------------------------------

def get_rulebook_subm(zIndices, zPtr, batchSize, spatialShape, outSpatialShape, kernelSize, stride,
                      padding, dilation, tileSize=None) -> RuleBook:
    """Fast form of :func:`get_rules_subm`: the compact rule book only."""
    if any(int(s) != 1 for s in stride):
        raise L.SphconvError("submanifold convolution needs stride 1, got %s" % (list(stride),))
    if list(map(int, spatialShape)) != list(map(int, outSpatialShape)):
        raise L.SphconvError("submanifold convolution keeps the spatial shape")
    return RuleBook.build_subm(zIndices, zPtr, batchSize, spatialShape, kernelSize, padding, dilation)


def get_rulebook(zIndices, zPtr, batchSize, spatialShape, outSpatialShape, kernelSize, stride,
                 padding, dilation, tileSize=None) -> RuleBook:
    """Fast form of :func:`get_rules`."""
    return RuleBook.build(zIndices, zPtr, batchSize, spatialShape, outSpatialShape, kernelSize,
                          stride, padding, dilation)


def get_rules_subm(zIndices, zPtr, batchSize, spatialShape, outSpatialShape, kernelSize, stride,
                   padding, dilation, tileSize) -> List[torch.Tensor]:
    """rules.cu:326-390 -> [zIndices, zPtr, rules, ruleSize] (the input index
    tensors are returned as they are, rules.cu:389)."""
    book = get_rulebook_subm(zIndices, zPtr, batchSize, spatialShape, outSpatialShape, kernelSize,
                             stride, padding, dilation)
    rules, rule_size = book.padded(tileSize)
    return [zIndices, zPtr, rules, rule_size]


def get_rules(zIndices, zPtr, batchSize, spatialShape, outSpatialShape, kernelSize, stride,
              padding, dilation, tileSize) -> List[torch.Tensor]:
    """rules.cu:405-486 -> [ozIndices, ozPtr, rules, ruleSize]."""
    book = get_rulebook(zIndices, zPtr, batchSize, spatialShape, outSpatialShape, kernelSize, stride,
                        padding, dilation)
    rules, rule_size = book.padded(tileSize)
    return [book.oz_idx, book.oz_ptr, rules, rule_size]


# ---- rule_conv.h ------------------------------------------------------------

def _check_conv_args(feature, weight):
    if feature.dim() != 2 or weight.dim() != 3 or feature.shape[1] != weight.shape[1]:
        raise L.SphconvError("feature [N,iC] / weight [KV,iC,oC] mismatch: %s vs %s"
                             % (tuple(feature.shape), tuple(weight.shape)))
    if weight.dtype != feature.dtype:
        weight = weight.to(feature.dtype)
    return weight


def rule_conv(feature: torch.Tensor, weight: torch.Tensor, rules, ruleSize, outNNZ: int,
              scale: Optional[torch.Tensor] = None, shift: Optional[torch.Tensor] = None,
              relu: bool = False, packed: Optional[torch.Tensor] = None, cache_packed: bool = False) -> torch.Tensor:
    """rule_conv.cu:286-336: out[j] = sum over pairs (k,i,j) feature[i] @ weight[k].
    ``scale``/``shift`` (fp32 [oC]) and ``relu`` fuse y = relu(acc*scale + shift)
    into the store (no reference counterpart; default off).  ``packed``: the
    fragment-ordered copy of this very ``weight`` that ``RuleBook.build*(..., weight=)``
    returned, which saves the packing launch; ``cache_packed``: keep the copy made here with the weight
    (see :func:`_packed_weight`).  A RuleBook made with ``lazy=True`` gets its pairs generated by the same
    launch that convolves them (``RuleBook.fused_forward``) where that is the faster way."""
    weight = _check_conv_args(feature, weight)
    book = _as_book(rules, ruleSize, feature.shape[0], int(outNNZ))
    if book.out_rows != int(outNNZ) or book.kv != weight.shape[0]:
        raise L.SphconvError("rules hold %d output rows / %d offsets, call says %d / %d"
                             % (book.out_rows, book.kv, int(outNNZ), weight.shape[0]))
    if packed is None:
        packed = _packed_weight(weight, False, cache=cache_packed)
    elif packed.numel() != L.lib().sph_weight_packed_bytes(L.dtype_code(weight.dtype), weight.shape[0],
                                                           weight.shape[1], weight.shape[2]):
        raise L.SphconvError("packed weight of %d bytes does not belong to a weight of shape %s"
                             % (packed.numel(), tuple(weight.shape)))
    if not book.built and feature.is_cuda and feature.shape[0] == book.in_rows:
        epi = None
        if scale is not None or shift is not None or relu:
            epi = L.Epilogue(L.ptr(scale), L.ptr(shift), int(bool(relu)))
        out = book.fused_forward(feature, packed, weight.shape[1], weight.shape[2], epi)
        if out is not None:
            return out
    return _apply(feature, packed, weight.shape[1], weight.shape[2], _conv_buffers(book, feature, weight, False),
                  scale, shift, relu)


def _conv_buffers(book, feature, weight, transposed: bool):
    """The book's buffers for one convolution call; a book kept by rows only gets its groups built
    when this call cannot go by rows."""
    buf = book.transposed() if transposed else book.fwd
    if buf.groups:
        return buf
    es = feature.element_size()
    kdim, ndim = weight.shape[1], weight.shape[2]
    by_rows = (kdim * es) % 16 == 0 and kdim * es <= 128 and (ndim * es) % 16 == 0 and feature.data_ptr() % 16 == 0 \
        and feature.shape[0] > 0
    return buf if by_rows else book.grouped(transposed)


def rule_conv_int8(feature: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor, rules, ruleSize,
                   outNNZ: int) -> torch.Tensor:
    """int8 x int8 -> int32 accumulate -> int8 with per-output-channel scales:
    q = clamp(rint(float(acc) * scale[oc]), -128, 127), round half to even."""
    if feature.dtype != torch.int8 or weight.dtype != torch.int8:
        raise L.SphconvError("rule_conv_int8 needs int8 feature and weight")
    _check_conv_args(feature, weight)
    book = _as_book(rules, ruleSize, feature.shape[0], int(outNNZ))
    packed = _packed_weight(weight, False)
    scale = scale.to(torch.float32).contiguous()
    if not book.built and feature.is_cuda and feature.shape[0] == book.in_rows:
        out = book.fused_forward(feature, packed, weight.shape[1], weight.shape[2], L.Epilogue(L.ptr(scale), None, 0))
        if out is not None:
            return out
    return _apply(feature, packed, weight.shape[1], weight.shape[2], _conv_buffers(book, feature, weight, False), scale)


def rule_conv_d_feature(feature: torch.Tensor, weight: torch.Tensor, rules, ruleSize,
                        tile_grid_shape, outNNZ: int) -> torch.Tensor:
    """rule_conv.cu:520-575.  ``feature`` is d_out [outRows,oC], ``weight`` the
    forward weight permuted to [KV,oC,iC] (functional.py:73), ``outNNZ`` the number
    of input rows; returns d_feature [outNNZ,iC]."""
    weight = _check_conv_args(feature, weight)
    book = _as_book(rules, ruleSize, int(outNNZ), feature.shape[0])
    buf, reverse = _dgrad_buffers(book, feature, weight.shape[1], weight.shape[2])
    if buf is None:
        buf = _conv_buffers(book, feature, weight, True)
    packed = _packed_weight(weight, False, reverse)
    return _apply(feature, packed, weight.shape[1], weight.shape[2], buf)


def rule_conv_d_weight(feature: torch.Tensor, d_featureOut: torch.Tensor, rules, ruleSize,
                       out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """rule_conv.cu:469-518 -> d_weight [KV,iC,oC], reduced in fp32 and stored in the features' type, or in
    float32 with ``out_dtype=torch.float32`` (16-bit features with an fp32 master weight)."""
    book = _as_book(rules, ruleSize, feature.shape[0], d_featureOut.shape[0])
    feature = feature.contiguous()
    d_out = d_featureOut.contiguous()
    if d_out.dtype != feature.dtype:
        d_out = d_out.to(feature.dtype)
    lib = L.lib()
    ic, oc = feature.shape[1], d_out.shape[1]
    n = lib.sph_wgrad_partial_elems(book.kv, ic, oc, book.out_rows)
    partial = torch.empty(max(n, 1), dtype=torch.float32, device=feature.device)
    if out_dtype not in (None, feature.dtype, torch.float32):
        raise L.SphconvError("d_weight comes in the features' type or in float32, not %s" % out_dtype)
    f32 = out_dtype == torch.float32
    dw = torch.empty((book.kv, ic, oc), dtype=torch.float32 if f32 else feature.dtype, device=feature.device)
    b = book.grouped().struct()
    L.check(lib.sph_conv_wgrad(L.dtype_code(feature.dtype), L.ptr(feature), feature.shape[0], ic,
                               L.ptr(d_out), oc, C.byref(b), L.ptr(partial), L.ptr(dw), int(f32), L.stream()))
    return dw


def rule_conv_backward(d_featureOut: torch.Tensor, feature: torch.Tensor, weight: torch.Tensor, rules,
                       ruleSize, tile_grid_shape) -> List[torch.Tensor]:
    """rule_conv.cu:577-597 -> [d_feature, d_weight]; ``weight`` is [KV,oC,iC]."""
    book = _as_book(rules, ruleSize, feature.shape[0], d_featureOut.shape[0])
    d_out = d_featureOut.contiguous()
    if d_out.dtype != feature.dtype:
        d_out = d_out.to(feature.dtype)
    d_feature = rule_conv_d_feature(d_out, weight, book, None, tile_grid_shape, feature.shape[0])
    d_weight = rule_conv_d_weight(feature, d_out, book, None)
    return [d_feature, d_weight]
