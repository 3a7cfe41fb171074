"""Several scans in flight: rule generation + forward of one submanifold layer for a
stream of independent LiDAR scans, each scan on one of a few HIP streams.

No reference counterpart (the reference launches everything on the legacy default
stream, rule_conv.cu:139,333).  One 100k-voxel scan does not fill the chip, so the
kernels of the next scan run beside those of the current one; the work per scan is
unchanged.  All device memory (rule books, outputs) is allocated once, per stream slot;
the weight is put in MFMA fragment order when the pipeline is made and again by
``set_weight`` (a serving pipeline's weight changes when the model does, not per scan).
A scan of up to RuleBook.FUSED_MAX_TILES tiles takes ONE launch (rules + forward,
``sph_rules_conv``), a larger one two (``sph_rules_build``, ``sph_conv_apply``).
"""
import ctypes as C
from typing import List, Sequence, Tuple

import torch

from . import _lib as L
from .rulebook import RuleBook, _Buffers, _check_index_tensors, _row_cols_ptr


class ScanPipeline:
    """``submit(feature, z_idx, z_ptr)`` enqueues rules + forward of one scan on the next
    stream slot and returns ``(out, slot)``; ``out`` [n, oC] is a view of that slot's output
    buffer and is overwritten when the slot comes round again (after ``streams`` submits).
    Call ``wait(slot)`` (or ``synchronize()``) before reading it on another stream.
    Lifetime of the inputs: ``submit`` records their use on the slot's stream
    (``Tensor.record_stream``), so the caller may drop or rebind them as soon as it returns;
    it must not overwrite them in place before the slot's scan has finished (``wait``)."""

    def __init__(self, weight: torch.Tensor, batch: int, shape: Sequence[int], kernel: Sequence[int] = (3, 3, 3),
                 max_voxels: int = 1 << 18, streams: int = 3, fused: bool = True):
        if weight.dim() == 5:
            weight = weight.reshape(-1, weight.shape[3], weight.shape[4])
        if weight.dim() != 3 or not weight.is_cuda:
            raise L.SphconvError("weight must be a GPU tensor [KV,iC,oC] or [K0,K1,K2,iC,oC]")
        self.weight = weight.detach().contiguous()
        self.kv, self.ic, self.oc = (int(v) for v in self.weight.shape)
        self.kernel = [int(k) for k in kernel]
        if self.kernel[0] * self.kernel[1] * self.kernel[2] != self.kv:
            raise L.SphconvError("weight holds %d offsets, kernel %s has %d" % (self.kv, self.kernel,
                                 self.kernel[0] * self.kernel[1] * self.kernel[2]))
        self.batch, self.shape = int(batch), [int(v) for v in shape]
        self.max_voxels = int(max_voxels)
        self.dt = L.dtype_code(self.weight.dtype)
        dev = self.weight.device
        lib = L.lib()
        pad = [k // 2 for k in self.kernel]
        self._geom = L.make_geom(self.batch, self.shape, self.shape, self.kernel, (1, 1, 1), pad)
        nbytes = lib.sph_weight_packed_bytes(self.dt, self.kv, self.ic, self.oc)
        if nbytes == 0:
            raise L.SphconvError("cannot pack weight of shape %s" % (tuple(self.weight.shape),))
        self._epi = L.Epilogue(None, None, 0)
        self._streams = [torch.cuda.Stream(device=dev) for _ in range(int(streams))]
        self._books = [_Buffers(self.max_voxels, self.kv, dev) for _ in self._streams]
        # One launch per scan while a scan's tiles are resident at once; with three or more scans in flight the two
        # kernels overlap better from 768 tiles on (measured at 937 tiles on three streams: 24.7 against 25.9 us per scan)
        self._fused_max_tiles = 768 if len(self._streams) >= 3 else RuleBook.FUSED_MAX_TILES
        for book in self._books:
            book.struct().middle_run = 1              # submanifold: every row pairs with itself at the middle offset
        self._packed = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        self._packed_ready = torch.cuda.Event()
        self.fused = bool(fused)
        self._out = [torch.empty((self.max_voxels, self.oc), dtype=self.weight.dtype, device=dev) for _ in self._streams]
        self._done = [torch.cuda.Event() for _ in self._streams]
        self._next = 0
        self._lib = lib
        self.set_weight(self.weight)

    def set_weight(self, weight: torch.Tensor):
        """Takes (a new value of) the layer's weight: packs it on the caller's current stream; scans submitted
        afterwards wait for the copy.  Scans still in flight may see either value: ``synchronize()`` first if
        that matters."""
        if weight.dim() == 5:
            weight = weight.reshape(-1, weight.shape[3], weight.shape[4])
        if tuple(weight.shape) != (self.kv, self.ic, self.oc) or weight.dtype != self.weight.dtype:
            raise L.SphconvError("weight must stay [%d,%d,%d] %s" % (self.kv, self.ic, self.oc, self.weight.dtype))
        self.weight = weight.detach().contiguous()
        w = self.weight
        L.check(self._lib.sph_weight_pack(self.dt, w.data_ptr(), self.kv, self.ic, self.oc, self.ic * self.oc, self.oc, 1,
                                          self._packed.data_ptr(), L.stream()))
        self._packed_ready.record(torch.cuda.current_stream())
        self._packed_seen = [False] * len(self._streams)

    @property
    def streams(self) -> int:
        return len(self._streams)

    def submit(self, feature: torch.Tensor, z_idx: torch.Tensor, z_ptr: torch.Tensor,
               wait_inputs: bool = True, row_cols: torch.Tensor = None) -> Tuple[torch.Tensor, int]:
        """``wait_inputs=False`` skips making the slot's stream wait for the caller's current stream:
        only for inputs that are already complete (e.g. produced before a synchronisation, or on
        ``stream_of(slot)`` itself).  ``row_cols`` (optional, int32 [n]): the column of every row
        (``SparseConvTensor.row_cols``); saves the rule generation its search of ``z_ptr``."""
        n = int(z_idx.shape[0])
        if n > self.max_voxels:
            raise L.SphconvError("scan of %d voxels, pipeline sized for %d" % (n, self.max_voxels))
        if feature.shape != (n, self.ic) or feature.dtype != self.weight.dtype or not feature.is_contiguous():
            raise L.SphconvError("feature must be contiguous [%d,%d] %s" % (n, self.ic, self.weight.dtype))
        _check_index_tensors(z_idx, z_ptr, self.batch, self.shape)
        slot = self._next
        self._next = (slot + 1) % len(self._streams)
        side = self._streams[slot]
        if wait_inputs:
            side.wait_stream(torch.cuda.current_stream())   # the inputs were produced on the caller's stream
        if not self._packed_seen[slot]:
            side.wait_event(self._packed_ready)              # the packed weight was made on another stream
            self._packed_seen[slot] = True
        # the kernels below read the inputs on the slot's stream: tell the caching allocator, so that a caller
        # who drops or rebinds them right after this call does not get their memory handed out again while
        # those kernels still run
        for t in (feature, z_idx, z_ptr) + ((row_cols,) if row_cols is not None else ()):
            t.record_stream(side)
        st = side.cuda_stream
        book = self._books[slot]
        book._struct.rows = n                                 # the slot's buffers hold up to max_voxels rows
        lib = self._lib
        hint = _row_cols_ptr(row_cols, n)
        zi, zp = z_idx.data_ptr(), z_ptr.data_ptr()
        rc = L.ERR_UNSUPPORTED
        if self.fused and lib.sph_book_tiles(n) <= self._fused_max_tiles:
            rc = lib.sph_rules_conv(zi, zp, n, zi, zp, n, C.byref(self._geom), C.byref(book._struct),
                                    L.FUSED_IN_FLIGHT if len(self._streams) >= 3 else 0, hint, self.dt,
                                    feature.data_ptr(), self.ic, self._packed.data_ptr(), self.oc, C.byref(self._epi),
                                    self._out[slot].data_ptr(), st)
        if rc == L.ERR_UNSUPPORTED:
            rc = lib.sph_rules_build(zi, zp, n, zi, zp, n, C.byref(self._geom), 0, C.byref(book._struct), hint, st)
            if rc == 0:
                rc = lib.sph_conv_apply(self.dt, feature.data_ptr(), n, self.ic, self._packed.data_ptr(), self.oc,
                                        C.byref(book._struct), C.byref(self._epi), self._out[slot].data_ptr(), st)
        if rc:
            L.check(rc)
        self._done[slot].record(side)
        return self._out[slot][:n], slot

    def launches_for(self, n: int) -> int:
        """Kernel launches ``submit`` makes for a scan of ``n`` voxels: 1 (rules + forward together) or 2."""
        return 1 if self.fused and self._lib.sph_book_tiles(int(n)) <= self._fused_max_tiles else 2

    def next_slot(self) -> int:
        return self._next

    def stream_of(self, slot: int) -> torch.cuda.Stream:
        """The slot's stream, for producers that want to enqueue a scan's inputs where it will be used."""
        return self._streams[slot]

    def wait(self, slot: int):
        """Makes the caller's current stream wait for the scan last submitted to ``slot``."""
        torch.cuda.current_stream().wait_event(self._done[slot])

    def synchronize(self):
        for s in self._streams:
            s.synchronize()
