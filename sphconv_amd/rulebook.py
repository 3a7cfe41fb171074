"""Rule book: this package's compact form of the reference's rule tensors.

The reference returns ``rules [NTile,KV,2,tile_n_max]`` padded with -1 plus
``rule_size [NTile,KV]`` (src/sphconv/rules.cu:364-369): hundreds of megabytes of
padding at LiDAR sizes.  A :class:`RuleBook` keeps the same pairs in the layout
the HIP kernels consume (see ``include/sphconv_hip.h``) and materialises the
padded tensors only when asked (:meth:`RuleBook.padded`).
"""
import ctypes as C
from typing import List, Optional, Sequence

import torch

from . import _lib as L


class _Buffers:
    """Device arrays of one book (forward or transposed), carved out of ONE allocation
    (a single caching-allocator call per book); the named tensors are views made on
    first access."""

    _FIELDS = ("tile_ngrp", "tile_koff", "grp_k", "grp_gather", "grp_owner", "tile_nbr")

    def __init__(self, rows: int, kv: int, device, by_row: bool = False, groups: bool = True):
        """``by_row`` also keeps the pairs by stationary row (``tile_nbr`` [NT,KV,128]), the form the
        convolution walks when neighbourhoods are dense; with it, ``groups=False`` leaves the groups out
        (forward-only use: the rule kernel then writes a fifth of the bytes)."""
        lib = L.lib()
        self.rows, self.kv = int(rows), int(kv)
        self.ntiles = lib.sph_book_tiles(self.rows)
        self.cap = lib.sph_book_cap(self.kv)
        self.by_row = bool(by_row)
        self.groups = bool(groups) or not self.by_row
        nt = max(self.ntiles, 1)
        g = 1 if self.groups else 0
        sizes = (nt * 4, nt * (self.kv + 1) * 2, g * nt * self.cap * 4, g * nt * self.cap * L.GROUP * 4,
                 g * nt * self.cap * L.GROUP * 4, nt * self.kv * L.TILE_ROWS * 4 if by_row else 0)
        self._off = []
        total = 0
        for sz in sizes:
            self._off.append(total)
            total += (sz + 255) & ~255
        self._sizes = sizes
        self.storage = torch.empty(total, dtype=torch.uint8, device=device)
        base = self.storage.data_ptr()
        ptrs = [base + o for o in self._off]
        if not self.groups:
            ptrs[2] = ptrs[3] = ptrs[4] = None
        self._struct = L.Book(*ptrs[:5], self.rows, self.kv, ptrs[5] if by_row else None, 0)
        self._views = {}

    def struct(self) -> L.Book:
        return self._struct

    def __getattr__(self, name):
        # views of the single allocation, typed and shaped like the C arrays
        if name in _Buffers._FIELDS:
            v = self._views.get(name)
            if v is None:
                i = _Buffers._FIELDS.index(name)
                raw = self.storage[self._off[i]:self._off[i] + self._sizes[i]]
                v = raw.view(torch.int16 if name == "tile_koff" else torch.int32)
                if name == "tile_koff":
                    v = v.view(max(self.ntiles, 1), self.kv + 1)
                if name == "tile_nbr":
                    v = v.view(max(self.ntiles, 1), self.kv, L.TILE_ROWS) if self.by_row else None
                elif name.startswith("grp_") and not self.groups:
                    v = None
                self._views[name] = v
            return v
        raise AttributeError(name)

    def num_pairs(self) -> int:
        """Total pairs held (synchronises)."""
        if self.ntiles == 0:
            return 0
        if not self.groups:
            return int((self.tile_nbr[:self.ntiles] >= 0).sum().item())
        ng = self.tile_ngrp[:self.ntiles].long()
        own = self.grp_owner.view(self.ntiles, self.cap * L.GROUP)
        used = torch.arange(self.cap * L.GROUP, device=own.device)[None, :] < (ng * L.GROUP)[:, None]
        return int(((own >= 0) & used).sum().item())


_NO_EPILOGUE = L.Epilogue(None, None, 0)

# Estimated pairs per stationary row from which a book also keeps its pairs by row (and the
# convolution walks that form).  float("inf") never does, 0 always.
BY_ROW_MIN_PAIRS = 10.0
# A book built for a forward pass that is known to go by rows, with no gradient being recorded, leaves
# its groups out (a fifth of the bytes the rule kernel writes), which moves the break-even down:
# measured on a 4x32x1024x32 grid, rules + convolution, by rows against by groups: 153/155 us at an
# estimate of 5.4 pairs per row, 177/205 at 6.75, 215/285 at 8.1 (32->32 fp16); 358/325, 432/460,
# 502/598 (64->64).  The threshold of such books is this fraction of the one above.
BY_ROW_FORWARD_ONLY = 0.65


class RuleBook:
    """Pairs of one convolution geometry on one sparse tensor."""

    def __init__(self, z_idx, z_ptr, oz_idx, oz_ptr, batch, in_shape, out_shape, kernel, stride,
                 padding, dilation, subm, row_cols=None, out_row_cols=None):
        self.z_idx, self.z_ptr = z_idx, z_ptr
        self.oz_idx, self.oz_ptr = oz_idx, oz_ptr
        # optional: the column of every input / output row (what init_tensor and the output-coordinate kernels know
        # when they write the rows); the rule kernel then need not search z_ptr for them
        self.row_cols, self.out_row_cols = row_cols, out_row_cols
        self.batch = int(batch)
        self.in_shape = [int(v) for v in in_shape]
        self.out_shape = [int(v) for v in out_shape]
        self.kernel = [int(v) for v in kernel]
        self.stride = [int(v) for v in stride]
        self.padding = [int(v) for v in padding]
        self.dilation = [int(v) for v in dilation]
        self.subm = bool(subm)
        self.kv = self.kernel[0] * self.kernel[1] * self.kernel[2]
        self.in_rows = int(z_idx.shape[0]) if z_idx is not None else 0
        self.out_rows = int(oz_idx.shape[0]) if oz_idx is not None else 0
        self._fwd: Optional[_Buffers] = None   # built on first use (see ``fwd``)
        self._bwd: Optional[_Buffers] = None
        self.keep = True                       # a fused rules + forward launch also writes the book (``fused_forward``)
        # (input channels, output channels, element size) of the forward pass a lazy book is made for, when no
        # gradient will be asked of it: lets a book that goes by rows leave its groups out (see ``_build``)
        self.forward_only: Optional[tuple] = None
        self._padded = {}
        self._from_padded = None     # (rules, rule_size) when built from reference-format tensors

    # -- construction -----------------------------------------------------
    @property
    def fwd(self) -> _Buffers:
        """The forward book (stationary on output rows); a book made with ``lazy=True`` is built here."""
        if self._fwd is None:
            self._fwd = self._build(False)
        return self._fwd

    @fwd.setter
    def fwd(self, buf):
        self._fwd = buf

    @property
    def built(self) -> bool:
        return self._fwd is not None

    def geom(self) -> L.Geom:
        return L.make_geom(self.batch, self.in_shape, self.out_shape, self.kernel, self.stride,
                           self.padding, self.dilation)

    def _pairs_per_row(self, transposed: bool) -> float:
        """Pairs a stationary row can expect: kernel volume x occupancy of the gathered side's grid
        (a stride thins the offsets that can pair with an input row)."""
        rows, shape = (self.out_rows, self.out_shape) if transposed else (self.in_rows, self.in_shape)
        cells = max(self.batch * shape[0] * shape[1] * shape[2], 1)
        est = self.kv * rows / cells
        if transposed:
            est /= self.stride[0] * self.stride[1] * self.stride[2]
        return est

    def _rows_kernel_takes(self, weight, weight_transposed: bool) -> bool:
        """Whether ``sph_conv_apply`` can walk this layer by stationary row (rows of 16-byte multiples up
        to 128 bytes, 16-byte multiples out, a table that fits LDS): the conditions of the library."""
        kv, wa, wb = weight.shape
        kdim, ndim = (wb, wa) if weight_transposed else (wa, wb)
        return self._rows_kernel_takes_shape(kdim, ndim, weight.element_size())

    def _rows_kernel_takes_shape(self, kdim: int, ndim: int, es: int) -> bool:
        return (kdim * es) % 16 == 0 and kdim * es <= 128 and (ndim * es) % 16 == 0 and self.kv * L.TILE_ROWS * 4 <= 48 * 1024

    def _build(self, transposed: bool, weight=None, weight_transposed: bool = False, groups: Optional[bool] = None):
        """Launches the rule kernel.  With ``weight`` [KV,a,b] its fragment-ordered copy (what
        ``sph_weight_pack`` makes, for the contraction over ``a``, or over ``b`` when
        ``weight_transposed``) is produced by the same launch and returned with the buffers.
        ``groups`` None: a by-row book leaves its groups out when it is built for a forward pass that
        is known to go by rows and no gradient is being recorded (they are built on demand later:
        :meth:`grouped`)."""
        rows = self.in_rows if transposed else self.out_rows
        est = self._pairs_per_row(transposed)
        by_row = est >= BY_ROW_MIN_PAIRS
        if groups is None:
            forward_only = (weight is not None and not torch.is_grad_enabled() and weight.dim() == 3
                            and self._rows_kernel_takes(weight, weight_transposed))
            if weight is None and not transposed and self.forward_only is not None and not torch.is_grad_enabled():
                forward_only = self._rows_kernel_takes_shape(*self.forward_only)
            if forward_only:
                by_row = est >= BY_ROW_MIN_PAIRS * BY_ROW_FORWARD_ONLY
            groups = not (by_row and forward_only)
        buf = _Buffers(rows, self.kv, self.z_ptr.device, by_row, groups)
        buf.struct().middle_run = int(self.subm)     # every row pairs with itself at the middle offset
        g, b = self.geom(), buf.struct()
        lib = L.lib()
        hint = _row_cols_ptr(self.row_cols if transposed else self.out_row_cols, rows)
        if weight is None:
            rc = lib.sph_rules_build(self.z_idx.data_ptr(), self.z_ptr.data_ptr(), self.in_rows,
                                     self.oz_idx.data_ptr(), self.oz_ptr.data_ptr(), self.out_rows,
                                     C.byref(g), int(transposed), C.byref(b), hint, L.stream())
            if rc:
                L.check(rc)
            return buf
        w = weight.detach()
        if not w.is_contiguous():
            w = w.contiguous()
        if not w.is_cuda or w.dim() != 3:
            raise L.SphconvError("weight must be a GPU tensor [KV,iC,oC]")
        kv, wa, wb = w.shape
        kdim, ndim = (wb, wa) if weight_transposed else (wa, wb)
        skk, sn = (1, wb) if weight_transposed else (wb, 1)
        dt = L.dtype_code(w.dtype)
        nbytes = lib.sph_weight_packed_bytes(dt, kv, kdim, ndim)
        if nbytes == 0:
            raise L.SphconvError("cannot pack weight of shape %s" % (tuple(w.shape),))
        packed = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
        rc = lib.sph_rules_build_pack(self.z_idx.data_ptr(), self.z_ptr.data_ptr(), self.in_rows,
                                      self.oz_idx.data_ptr(), self.oz_ptr.data_ptr(), self.out_rows,
                                      C.byref(g), int(transposed), C.byref(b), hint, dt, w.data_ptr(), kv, kdim, ndim,
                                      wa * wb, skk, sn, packed.data_ptr(), L.stream())
        if rc:
            L.check(rc)
        return buf, packed

    @classmethod
    def build_subm(cls, z_idx, z_ptr, batch, shape, kernel, padding=None,
                   dilation=(1, 1, 1), weight=None, row_cols=None, lazy=False):
        """Submanifold rules (replaces get_rules_subm, rules.cu:326-390): stride 1,
        outputs are the inputs; ``padding`` defaults to K//2 (conv.py:210).
        With ``weight`` [KV,iC,oC] returns ``(book, packed_weight)``: the layer's weight is
        put in fragment order by the same kernel launch (pass it to ``rule_conv(..., packed=)``).
        ``row_cols`` (optional, int32 [NNZ]): the column of every row (``SparseConvTensor.row_cols``).
        ``lazy``: launch nothing yet; the pairs are generated by the first use -- by ``rule_conv`` in the same
        launch as the convolution where the library has that kernel (:meth:`fused_forward`)."""
        _check_index_tensors(z_idx, z_ptr, batch, shape)
        pad = [int(k) // 2 for k in kernel] if padding is None else [int(v) for v in padding]
        rb = cls(z_idx, z_ptr, z_idx, z_ptr, batch, shape, shape, kernel, (1, 1, 1), pad, dilation, True,
                 row_cols, row_cols)
        if lazy:
            return rb
        if weight is None:
            rb.fwd = rb._build(False)
            return rb
        rb.fwd, packed = rb._build(False, weight)
        return rb, packed

    @classmethod
    def count_ahead(cls, z_idx, z_ptr, batch, in_shape, out_shape, kernel, stride, padding, dilation=(1, 1, 1)):
        """First half of :meth:`build`, to be enqueued as soon as a strided layer's INPUT coordinates exist:
        the output rows per column are counted and scanned, the row count goes to pinned host memory, and an
        event marks the place in the stream.  Pass the returned object to ``build(..., ahead=)`` when the layer
        itself is reached: whatever the caller has enqueued in between (the convolutions of the layers before)
        keeps the GPU busy while the host reads the count, instead of the GPU waiting for the host."""
        _check_index_tensors(z_idx, z_ptr, batch, in_shape)
        lib = L.lib()
        dev = z_ptr.device
        g = L.make_geom(batch, in_shape, out_shape, kernel, stride, padding, dilation)
        if min(int(v) for v in out_shape) <= 0:
            raise L.SphconvError("empty output grid %s" % (list(out_shape),))
        nints = lib.sph_outcoords_scratch_ints(C.byref(g))
        if nints < 0:
            L.check(nints)
        oz_ptr = torch.empty((int(batch), int(out_shape[0]), int(out_shape[1])), dtype=torch.int32, device=dev)
        # scratch and the pinned word are this call's own: other strided layers may be generated before build()
        scratch = torch.empty(max(nints + (nints & 1), 2), dtype=torch.int32, device=dev)
        total = _pinned_word()
        stream = torch.cuda.current_stream(dev)
        L.check(lib.sph_outcoords_count(L.ptr(z_idx), L.ptr(z_ptr), int(z_idx.shape[0]), C.byref(g), L.ptr(oz_ptr),
                                        L.ptr(scratch), total.data_ptr(), stream.cuda_stream))
        event = torch.cuda.Event()
        event.record(stream)
        key = (z_idx.data_ptr(), z_ptr.data_ptr(), int(batch), tuple(int(v) for v in in_shape),
               tuple(int(v) for v in out_shape), tuple(int(v) for v in kernel), tuple(int(v) for v in stride),
               tuple(int(v) for v in padding), tuple(int(v) for v in dilation))
        return _CountAhead(key, oz_ptr, scratch, total, event, stream.cuda_stream)

    @classmethod
    def build(cls, z_idx, z_ptr, batch, in_shape, out_shape, kernel, stride, padding,
              dilation=(1, 1, 1), weight=None, ahead=None, row_cols=None, lazy=False):
        """Strided rules (replaces get_rules, rules.cu:405-486): output coordinates
        (oz_ptr inclusive scan, oz_idx ascending per column) and pairs.  One wait for the
        output row count, as in the reference (rules.cu:461): the count kernel writes it to pinned
        host memory, so the wait is a stream synchronisation and no copy.  ``ahead``: what
        :meth:`count_ahead` returned for the same arguments on the same stream; the wait is then for its
        event only."""
        _check_index_tensors(z_idx, z_ptr, batch, in_shape)
        lib = L.lib()
        dev = z_ptr.device
        g = L.make_geom(batch, in_shape, out_shape, kernel, stride, padding, dilation)
        if min(int(v) for v in out_shape) <= 0:
            raise L.SphconvError("empty output grid %s" % (list(out_shape),))
        n_in = int(z_idx.shape[0])
        stream = torch.cuda.current_stream(dev)
        if ahead is not None:
            key = (z_idx.data_ptr(), z_ptr.data_ptr(), int(batch), tuple(int(v) for v in in_shape),
                   tuple(int(v) for v in out_shape), tuple(int(v) for v in kernel), tuple(int(v) for v in stride),
                   tuple(int(v) for v in padding), tuple(int(v) for v in dilation))
            if ahead.key != key or ahead.stream != stream.cuda_stream:
                raise L.SphconvError("count_ahead() was called for another layer, tensor or stream")
            oz_ptr, scratch, total = ahead.oz_ptr, ahead.scratch, ahead.total
            ahead.event.synchronize()
        else:
            nints = lib.sph_outcoords_scratch_ints(C.byref(g))
            if nints < 0:
                L.check(nints)
            oz_ptr = torch.empty((int(batch), int(out_shape[0]), int(out_shape[1])), dtype=torch.int32, device=dev)
            scratch, total = _outcoords_workspace(dev, nints)
            try:
                # one launch: counts, their scan into oz_ptr, and the row count written straight to pinned host memory
                L.check(lib.sph_outcoords_count(L.ptr(z_idx), L.ptr(z_ptr), n_in, C.byref(g), L.ptr(oz_ptr),
                                                L.ptr(scratch), total.data_ptr(), stream.cuda_stream))
                stream.synchronize()             # the one wait of a strided layer (the reference's is rules.cu:461)
            except Exception:
                _WORKSPACES.pop(_workspace_key(dev), None)   # whatever failed, the next call starts from fresh buffers
                raise
        out_rows = int(total[0])
        oz_idx = torch.empty(out_rows, dtype=torch.int32, device=dev)
        out_cols = torch.empty(out_rows, dtype=torch.int32, device=dev)   # the output rows' columns, a by-product
        L.check(lib.sph_outcoords_fill(L.ptr(z_idx), L.ptr(z_ptr), n_in, C.byref(g), L.ptr(scratch),
                                       L.ptr(oz_ptr), L.ptr(oz_idx), out_rows, L.ptr(out_cols), L.stream()))
        if ahead is not None:
            _release_pinned_word(total)
        rb = cls(z_idx, z_ptr, oz_idx, oz_ptr, batch, in_shape, out_shape, kernel, stride, padding,
                 dilation, False, row_cols, out_cols)
        if lazy:                                     # output coordinates now, pairs with the first use
            return rb
        if weight is None:
            rb.fwd = rb._build(False)
            return rb
        rb.fwd, packed = rb._build(False, weight)    # (book, packed weight) as in build_subm
        return rb, packed

    @classmethod
    def from_padded(cls, rules, rule_size, in_rows: int, out_rows: int) -> "RuleBook":
        """Book from the reference's padded tensors (any tile size)."""
        if rules.dim() != 4 or rules.shape[2] != 2 or rule_size.dim() != 2 \
                or rule_size.shape[0] != rules.shape[0] or rule_size.shape[1] != rules.shape[1]:
            raise L.SphconvError("rules must be [NTile,KV,2,n] and rule_size [NTile,KV], got %s, %s"
                                 % (tuple(rules.shape), tuple(rule_size.shape)))
        if rules.dtype != torch.int32 or rule_size.dtype != torch.int32:
            raise L.SphconvError("rules and rule_size must be int32")
        rb = cls.__new__(cls)
        rb.z_idx = rb.z_ptr = rb.oz_idx = rb.oz_ptr = None
        rb.batch = 0
        rb.in_shape = rb.out_shape = rb.kernel = rb.stride = rb.padding = rb.dilation = None
        rb.subm = False
        rb.kv = int(rules.shape[1])
        rb.in_rows, rb.out_rows = int(in_rows), int(out_rows)
        rb._bwd = None
        rb._fwd = None
        rb.keep = True
        rb.forward_only = None
        rb.row_cols = rb.out_row_cols = None
        rb._padded = {}
        rb._from_padded = (rules.contiguous(), rule_size.contiguous())
        rb.fwd = rb._convert(False)
        return rb

    def _convert(self, transposed: bool) -> _Buffers:
        rules, rule_size = self._from_padded
        rows = self.in_rows if transposed else self.out_rows
        buf = _Buffers(rows, self.kv, rules.device)
        nbr = torch.empty(max(rows, 1) * self.kv, dtype=torch.int32, device=rules.device)
        b = buf.struct()
        L.check(L.lib().sph_rules_from_padded(L.ptr(rules), L.ptr(rule_size), int(rules.shape[0]),
                                              self.kv, int(rules.shape[3]), self.in_rows,
                                              self.out_rows, int(transposed), L.ptr(nbr),
                                              C.byref(b), L.stream()))
        return buf

    # Tiles up to which one launch for rules + forward beats two (three workgroups of four waves, or four of two,
    # per CU hold that many at once; beyond, the launch runs in rounds and the two kernels are as fast or faster:
    # measured on the 64 x 2048 x 64 grid, 64 -> 64 fp16: 746 tiles 21.8 against 26.1 us, 937 tiles 29.3 / 32.0,
    # 2457 tiles 68.6 / 66.9, 5957 tiles 140 / 142).
    FUSED_MAX_TILES = 1024

    def fused_forward(self, feature: torch.Tensor, packed: torch.Tensor, kdim: int, ndim: int, epilogue=None,
                      out: Optional[torch.Tensor] = None, buffers: Optional[_Buffers] = None):
        """Pairs and forward convolution of this (not yet built) book in ONE launch (``sph_rules_conv``): replaces
        get_rules_subm / get_rules' pair half + rule_conv (rules.cu:326-486, rule_conv.cu:286-336) where the
        reference launches three kernels.  Returns the output rows, or None when this layer is better served by
        the two kernels (dense neighbourhoods that go by rows, more than FUSED_MAX_TILES tiles, shapes the
        library's fused kernel does not take).  With ``self.keep`` the book is written too and the object counts
        as built afterwards; without, only the output exists and a later use of the book generates it."""
        if self._fwd is not None or self._from_padded is not None:
            return None
        lib = L.lib()
        es = feature.element_size()
        ntiles = lib.sph_book_tiles(self.out_rows)
        if self.out_rows == 0 or ntiles > self.FUSED_MAX_TILES or self.kv > 32 or ndim > 64 \
                or (kdim * es) % 16 or kdim * es > 128 or self._pairs_per_row(False) >= BY_ROW_MIN_PAIRS * BY_ROW_FORWARD_ONLY:
            return None
        if not feature.is_contiguous():
            feature = feature.contiguous()
        if buffers is not None:
            buf = buffers
        elif self.keep:
            buf = _Buffers(self.out_rows, self.kv, self.z_ptr.device)
        else:
            buf = _scratch_book(self.out_rows, self.kv, self.z_ptr.device)   # nobody keeps it: the stream's own
        buf.struct().middle_run = int(self.subm)
        if out is None:
            out = torch.empty((self.out_rows, ndim), dtype=feature.dtype, device=feature.device)
        g = self.geom()
        epi = epilogue if epilogue is not None else _NO_EPILOGUE
        rc = lib.sph_rules_conv(self.z_idx.data_ptr(), self.z_ptr.data_ptr(), self.in_rows, self.oz_idx.data_ptr(),
                                self.oz_ptr.data_ptr(), self.out_rows, C.byref(g), C.byref(buf.struct()), int(self.keep),
                                _row_cols_ptr(self.out_row_cols, self.out_rows), L.dtype_code(feature.dtype),
                                feature.data_ptr(), int(kdim), packed.data_ptr(), int(ndim), C.byref(epi), out.data_ptr(),
                                L.stream())
        if rc == L.ERR_UNSUPPORTED:
            return None
        if rc:
            L.check(rc)
        if self.keep:
            self._fwd = buf
        return out

    # -- views ------------------------------------------------------------
    def grouped(self, transposed: bool = False) -> _Buffers:
        """The forward (or transposed) book with its groups, which wgrad, the padded tensors and the
        grouped convolution kernels need; rebuilt once if it was made for a by-row forward pass only."""
        buf = self.transposed() if transposed else self.fwd
        if not buf.groups:
            buf = self._build(transposed, groups=True)
            if transposed:
                self._bwd = buf
            else:
                self._fwd = buf
        return buf

    def mirrored(self) -> bool:
        """True if the book is its own transpose up to mirroring the offsets (k <-> KV-1-k): submanifold,
        stride 1, odd kernel, padding K//2 -- then dgrad runs on the forward book with reversed weights."""
        return bool(self.subm and self.kernel is not None and self.oz_idx is self.z_idx
                    and all(k % 2 == 1 for k in self.kernel) and all(s == 1 for s in self.stride)
                    and all(p == k // 2 for p, k in zip(self.padding, self.kernel)))

    def transposed(self) -> _Buffers:
        """Book stationary on input rows (what dgrad gathers through when the book is not mirrored)."""
        if self._bwd is None:
            self._bwd = self._convert(True) if self._from_padded is not None else self._build(True)
        return self._bwd

    def num_pairs(self) -> int:
        return self.fwd.num_pairs()

    def padded(self, tile_size: Sequence[int] = (2, 2)):
        """-> (rules [NTile,KV,2,tile_n_max], rule_size [NTile,KV]) in the reference's
        format, lists in ascending output row.  ``tile_n_max`` is the reference's
        heuristic (rules.cu:21-28) raised, if needed, to the longest list so that no
        pair is dropped (the reference drops them, rules.cu:301-308)."""
        if self._from_padded is not None:
            return self._from_padded
        key = (int(tile_size[0]), int(tile_size[1]))
        if key not in self._padded:
            lib = L.lib()
            g, b = self.geom(), self.grouped().struct()
            dev = self.z_ptr.device
            ntile = lib.sph_num_tiles(C.byref(g), *key)
            nbr = torch.empty(max(self.out_rows, 1) * self.kv, dtype=torch.int32, device=dev)
            rule_size = torch.empty((ntile, self.kv), dtype=torch.int32, device=dev)
            L.check(lib.sph_rules_to_padded_count(C.byref(b), L.ptr(self.oz_ptr), C.byref(g), key[0],
                                                  key[1], L.ptr(nbr), L.ptr(rule_size), L.stream()))
            n_max = lib.sph_tile_n_max(C.byref(g), key[0], key[1], self.in_rows)
            longest = int(rule_size.max().item()) if rule_size.numel() else 0
            n_max = max(n_max, (longest + 15) & ~15, 16)
            rules = torch.empty((ntile, self.kv, 2, n_max), dtype=torch.int32, device=dev)
            L.check(lib.sph_rules_to_padded_fill(L.ptr(self.oz_ptr), C.byref(g), key[0], key[1],
                                                 L.ptr(nbr), self.out_rows, self.kv, n_max,
                                                 L.ptr(rules), L.stream()))
            self._padded[key] = (rules, rule_size)
        return self._padded[key]

    def tile_grid_shape(self, tile_size: Sequence[int] = (2, 2)) -> List[int]:
        """conv.py:32-38"""
        return [-(-self.out_shape[0] // int(tile_size[0])), -(-self.out_shape[1] // int(tile_size[1]))]


# Scratch of the output-coordinate kernels, kept per (device, stream), and one pinned host int that receives
# the output row count.
_WORKSPACES = {}


def _workspace_key(dev):
    dev = torch.device(dev)
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    return (index, torch.cuda.current_stream(index).cuda_stream)


# The scratch holds 8 bytes per output column and 64 bins (up to 128 MB, see sph_outcoords_count): it scales with
# the dense column grid, not with the number of voxels.  Up to this many int32 entries it is kept per (device,
# stream) between calls; a larger one belongs to its call and goes back to the allocator with it.
_WORKSPACE_KEEP_INTS = 1 << 24      # 64 MB


def _outcoords_workspace(dev, nints: int):
    key = _workspace_key(dev)
    ws = _WORKSPACES.get(key)
    if nints > _WORKSPACE_KEEP_INTS:
        total = ws[1] if ws is not None else torch.zeros(1, dtype=torch.int32).pin_memory()
        if ws is None:
            _WORKSPACES[key] = (torch.empty(1 << 16, dtype=torch.int32, device=dev), total)
        return torch.empty(nints + (nints & 1), dtype=torch.int32, device=dev), total
    if ws is None or ws[0].numel() < nints:
        scratch = torch.empty(max(nints + (nints & 1), 1 << 16), dtype=torch.int32, device=dev)
        total = ws[1] if ws is not None else torch.zeros(1, dtype=torch.int32).pin_memory()
        ws = (scratch, total)
        _WORKSPACES[key] = ws
    return ws


class _CountAhead:
    """Output-row counts of a strided layer on their way (RuleBook.count_ahead)."""

    def __init__(self, key, oz_ptr, scratch, total, event, stream):
        self.key, self.oz_ptr, self.scratch, self.total, self.event, self.stream = key, oz_ptr, scratch, total, event, stream


# Pinned host words that receive row counts; handed out one per count in flight and taken back when read
# (pinning memory costs a system call, so they are never freed).
_PINNED_WORDS = []


def _pinned_word():
    return _PINNED_WORDS.pop() if _PINNED_WORDS else torch.zeros(1, dtype=torch.int32).pin_memory()


def _release_pinned_word(word):
    if len(_PINNED_WORDS) < 64:
        _PINNED_WORDS.append(word)


# Scratch books of one-launch calls that keep no book (the kernel still wants one for tiles with more groups than
# its LDS holds): one per device, stream and kernel volume, grown on demand.  Calls on one stream run one after the
# other, so they can share it; calls on different streams get different ones.
_SCRATCH_BOOKS = {}


def _scratch_book(rows: int, kv: int, device) -> "_Buffers":
    key = (device.index, L.stream(), kv)
    buf = _SCRATCH_BOOKS.get(key)
    if buf is None or buf.capacity < rows:
        if len(_SCRATCH_BOOKS) >= 64:
            _SCRATCH_BOOKS.clear()
        buf = _Buffers(max(rows, 1 << 17), kv, device)
        buf.capacity = buf.rows
        _SCRATCH_BOOKS[key] = buf
    buf.struct().rows = rows
    return buf


def _row_cols_ptr(row_cols, rows: int):
    """Device pointer of a table of the rows' columns, or None when there is none (or it does not fit)."""
    if row_cols is None or not row_cols.is_cuda or row_cols.dtype != torch.int32 or not row_cols.is_contiguous() \
            or row_cols.dim() != 1 or row_cols.shape[0] != rows:
        return None
    return row_cols.data_ptr()


def row_columns(z_ptr: torch.Tensor, rows: int) -> torch.Tensor:
    """int32 [rows]: the column (index into the flattened ``z_ptr``) of every row."""
    out = torch.empty(int(rows), dtype=torch.int32, device=z_ptr.device)
    L.check(L.lib().sph_row_columns(L.ptr(z_ptr), z_ptr.numel(), int(rows), L.ptr(out), L.stream()))
    return out


def _check_index_tensors(z_idx, z_ptr, batch, shape):
    if z_idx.dtype != torch.int32 or z_ptr.dtype != torch.int32:
        raise L.SphconvError("z_idx and z_ptr must be int32")
    if z_idx.dim() != 1:
        raise L.SphconvError("z_idx must be [NNZ]")
    want = (int(batch), int(shape[0]), int(shape[1]))
    if tuple(z_ptr.shape) != want:
        raise L.SphconvError("z_ptr must be [B,S0,S1] = %s, got %s" % (want, tuple(z_ptr.shape)))
    if not (z_idx.is_contiguous() and z_ptr.is_contiguous()):
        raise L.SphconvError("z_idx and z_ptr must be contiguous")
    if not (z_idx.is_cuda and z_ptr.is_cuda):
        raise L.SphconvError("z_idx and z_ptr must be GPU tensors")
