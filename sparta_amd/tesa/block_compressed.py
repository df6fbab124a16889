"""Block-compressed (BCSR / BCSC / both) indexes on the GPU.

Host side of the index builder and of the dense<->compressed converters; the
device side is libsparta_hip (spx_bcs_index / spx_bcs_gather / spx_bcs_scatter /
spx_bcs_sum).  Mirrors the classes and attributes of
sparta/tesa/block_compressed.py:23-413 with two deliberate differences:

* entries are in canonical order (columns ascending inside a block-row for
  BCSR, rows ascending inside a block-column for BCSC) - one of the orders the
  reference's atomics may produce, but the same on every run;
* the number of live blocks stays on the device after a build.  `block_nnz`,
  `nnz`, `BCSR_idx` and `BCSC_idx` fetch it on first use (one synchronisation,
  cached), kernels that only walk `row_ptr` / `col_ptr` never need it.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from sparta_amd import _lib
from sparta_amd.tesa.tesa_base import TeSAIndexes, TeSAFunctionContext

_VALID_EDGES = (4, 8, 16, 32, 64, 128, 256)


class BCSIndexes(TeSAIndexes):
    """Common part of the three index flavours."""

    #: which array orders the compressed values ('bcsr' or 'bcsc')
    _value_order = 'bcsr'

    def __init__(self, function_context: 'BCSFunctionContext', raw_mask: torch.Tensor,
                 block_H: int, block_W: int, nnz_dev: torch.Tensor, capacity: int):
        super().__init__(function_context, raw_mask)
        self.block_H = block_H
        self.block_W = block_W
        self.H, self.W = raw_mask.shape
        self.row_num = self.H // block_H
        self.col_num = self.W // block_W
        self.capacity = capacity
        self.nnz_dev = nnz_dev
        self._block_nnz: Optional[int] = None

    # ---- live block count ----------------------------------------------------
    @property
    def block_nnz(self) -> int:
        if self._block_nnz is None:
            self._block_nnz = int(self.nnz_dev.item())
        return self._block_nnz

    @property
    def nnz(self) -> np.int32:
        return np.int32(self.block_nnz)

    # ---- scheduling hint -----------------------------------------------------------
    def launch_order(self, by: str) -> torch.Tensor:
        """int32 permutation of the block rows (by='row') or block columns (by='col'),
        longest first; computed on the GPU once per index and cached."""
        cache = self.__dict__.setdefault('_launch_order', {})
        if by not in cache:
            ptr = self.row_ptr if by == 'row' else self.col_ptr
            n = ptr.numel() - 1
            order = torch.empty((n,), dtype=torch.int32, device=ptr.device)
            rc = _lib.load().spx_bcs_schedule(_lib.dev_ptr(ptr), n, _lib.dev_ptr(order),
                                              _lib.current_stream(ptr.device))
            _lib.check(rc, 'spx_bcs_schedule')
            cache[by] = order
        return cache[by]

    # ---- decoding --------------------------------------------------------------
    def _value_index(self) -> Tuple[torch.Tensor, int]:
        """(index buffer at capacity, idx_kind) that orders compressed values."""
        raise NotImplementedError

    def block_coordinates(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """(block_row, block_col) int64 tensors in value order."""
        raise NotImplementedError

    def get_block_mask(self) -> torch.Tensor:
        """Rebuild the uint8 [row_num, col_num] block mask from the index."""
        rows, cols = self.block_coordinates()
        grid = torch.zeros((self.row_num, self.col_num), dtype=torch.uint8, device=rows.device)
        grid[rows, cols] = 1
        return grid

    def is_block_uniform(self) -> bool:
        """True when every element of every live block is set in the raw mask, i.e. the
        element mask carries no information beyond the block index.  Computed once per
        index (one synchronising comparison) and cached."""
        cached = self.__dict__.get('_block_uniform')
        if cached is None:
            cached = bool(torch.equal(self.get_mask() != 0, self.raw_mask != 0))
            self.__dict__['_block_uniform'] = cached
        return cached

    def get_mask(self) -> torch.Tensor:
        grid = self.get_block_mask()
        full = grid.repeat_interleave(self.block_H, dim=0).repeat_interleave(self.block_W, dim=1)
        return full.contiguous()

    # ---- values ------------------------------------------------------------------
    def convert(self, dense: torch.Tensor, at_capacity: bool = False) -> torch.Tensor:
        """Dense [..., H, W] -> compressed [..., nnz*block_H*block_W].

        With `at_capacity` the result has room for `capacity` blocks, of which the
        first nnz are written; the launch reads nnz from device memory, so nothing
        synchronises with the host (for masks that change every step)."""
        idx, kind = self._value_index()
        if at_capacity:
            return self.function_context.convert(dense, idx, self.capacity, self.H, self.W, idx_kind=kind,
                                                 nnz_dev=self.nnz_dev)
        return self.function_context.convert(dense, idx, self.block_nnz, self.H, self.W, idx_kind=kind)

    def inverse(self, sparse_val: torch.Tensor) -> torch.Tensor:
        """Compressed [..., nnz*block_H*block_W] -> zero-filled dense [..., H, W]."""
        idx, kind = self._value_index()
        return self.function_context.inverse(sparse_val, idx, self.block_nnz, self.H, self.W, idx_kind=kind)

    def sum(self, sparse_val: torch.Tensor, axis: int = -1) -> torch.Tensor:
        """Sum compressed values along a dense axis (-1: over W, -2: over H)."""
        from_end = -axis if axis < 0 else sparse_val.dim() + 1 - axis
        if from_end not in (1, 2):
            raise ValueError(f'axis #{axis} is not sparsed, please use torch.sum() instead.')
        idx, kind = self._value_index()
        return self.function_context.block_sum(
            sparse_val, idx, kind, self.block_nnz, self.H, self.W, axis=0 if from_end == 1 else 1)


class BCSRIndexes(BCSIndexes):
    """row_ptr + BCSR_idx, BCSR_idx = (block_row << 16) | block_col."""

    def __init__(self, function_context, raw_mask, row_ptr, bcsr_buf, nnz_dev, block_H, block_W):
        super().__init__(function_context, raw_mask, block_H, block_W, nnz_dev, bcsr_buf.numel())
        self.row_ptr = row_ptr
        self._bcsr_buf = bcsr_buf

    @property
    def BCSR_idx(self) -> torch.Tensor:
        return self._bcsr_buf[:self.block_nnz]

    def _value_index(self):
        return self._bcsr_buf, _lib.IDX_BCSR_I32

    def block_coordinates(self):
        code = self.BCSR_idx.to(torch.int64)
        return code >> 16, code & 0xffff


class BCSCIndexes(BCSIndexes):
    """col_ptr + BCSC_idx, BCSC_idx = (block_col << 16) | block_row (int32)."""

    _value_order = 'bcsc'

    def __init__(self, function_context, raw_mask, col_ptr, bcsc_buf, nnz_dev, block_H, block_W):
        super().__init__(function_context, raw_mask, block_H, block_W, nnz_dev, bcsc_buf.numel())
        self.col_ptr = col_ptr
        self._bcsc_buf = bcsc_buf

    @property
    def BCSC_idx(self) -> torch.Tensor:
        return self._bcsc_buf[:self.block_nnz]

    def _value_index(self):
        return self._bcsc_buf, _lib.IDX_BCSC_I32

    def block_coordinates(self):
        code = self.BCSC_idx.to(torch.int64)
        return code & 0xffff, (code >> 16) & 0xffff


class BCSRCIndexes(BCSRIndexes):
    """Both orders; values follow the BCSR order and the int64 BCSC_idx carries
    the BCSR position of each block in its upper half."""

    def __init__(self, function_context, raw_mask, row_ptr, col_ptr, bcsr_buf, bcsc_buf, nnz_dev,
                 block_H, block_W):
        super().__init__(function_context, raw_mask, row_ptr, bcsr_buf, nnz_dev, block_H, block_W)
        self.col_ptr = col_ptr
        self._bcsc_buf = bcsc_buf

    @property
    def BCSC_idx(self) -> torch.Tensor:
        return self._bcsc_buf[:self.block_nnz]


class BCSFunctionContext(TeSAFunctionContext):
    """Index builder / converter for one (block_H, block_W, BCSR, BCSC) choice."""

    def __init__(self, block_H: int, block_W: int, BCSR: bool, BCSC: bool):
        assert block_H in _VALID_EDGES, f'invalid block height {block_H}'
        assert block_W in _VALID_EDGES, f'invalid block width {block_W}'
        assert BCSR or BCSC, 'at least one of BCSR / BCSC is required'
        _lib.load()
        self._block_H = block_H
        self._block_W = block_W
        self._block_size = block_H * block_W
        self._BCSR = BCSR
        self._BCSC = BCSC
        self._workspaces: Dict[Tuple[int, int], int] = {}

    # ---- index build ------------------------------------------------------------
    def _workspace(self, H: int, W: int, device) -> torch.Tensor:
        """Scratch of one index build.  Taken from torch's caching allocator at every
        build (only the byte count is cached): the allocator hands a block back out
        only in stream order, so two operators - or two streams - that rebuild masks
        of one shape at the same time never share the liveness / prefix buffers."""
        key = (H, W)
        nbytes = self._workspaces.get(key)
        if nbytes is None:
            nbytes = _lib.load().spx_bcs_index_workspace_bytes(H, W, self._block_H, self._block_W)
            assert nbytes > 0, f'mask shape ({H}, {W}) does not fit block ({self._block_H}, {self._block_W})'
            self._workspaces[key] = nbytes
        return torch.empty((nbytes,), dtype=torch.uint8, device=device)

    def _prepare(self, mask: torch.Tensor, capacity: Optional[int] = None) -> dict:
        """Output buffers and workspace of one index build (everything
        spx_bcs_index_scheduled takes), allocated but not yet filled."""
        assert mask.dim() == 2, 'only 2D mask is supported'
        if mask.dtype != torch.uint8:
            mask = (mask != 0).to(torch.uint8)
        mask = mask.contiguous()
        H, W = mask.shape
        BH, BW = self._block_H, self._block_W
        assert H % BH == 0 and W % BW == 0, f'mask shape ({H}, {W}) does not fit block ({BH}, {BW})'
        R, Cn = H // BH, W // BW
        cap = R * Cn if capacity is None else int(capacity)
        dev = mask.device
        i32 = dict(dtype=torch.int32, device=dev)
        job = dict(mask=mask, H=H, W=W, cap=cap, nnz_dev=torch.empty((1,), **i32),
                   row_ptr=None, bcsr=None, col_ptr=None, bcsc=None, row_order=None, col_order=None)
        if self._BCSR:
            job['row_ptr'] = torch.empty((R + 1,), **i32)
            job['bcsr'] = torch.empty((cap,), **i32)
            job['row_order'] = torch.empty((R,), **i32)   # the launch orders of the matmul kernels
        both = self._BCSR and self._BCSC
        if self._BCSC:
            job['col_ptr'] = torch.empty((Cn + 1,), **i32)
            job['bcsc'] = torch.empty((cap,), dtype=torch.int64 if both else torch.int32, device=dev)
            job['col_order'] = torch.empty((Cn,), **i32)  # come out of the same launch
        job['ws'] = self._workspace(H, W, dev)
        return job

    def _wrap(self, job: dict) -> BCSIndexes:
        BH, BW = self._block_H, self._block_W
        if self._BCSR and self._BCSC:
            indexes = BCSRCIndexes(self, job['mask'], job['row_ptr'], job['col_ptr'], job['bcsr'], job['bcsc'],
                                   job['nnz_dev'], BH, BW)
        elif self._BCSR:
            indexes = BCSRIndexes(self, job['mask'], job['row_ptr'], job['bcsr'], job['nnz_dev'], BH, BW)
        else:
            indexes = BCSCIndexes(self, job['mask'], job['col_ptr'], job['bcsc'], job['nnz_dev'], BH, BW)
        indexes.__dict__['_launch_order'] = {k: v for k, v in (('row', job['row_order']), ('col', job['col_order']))
                                             if v is not None}
        return indexes

    def build_indexes(self, mask: torch.Tensor, capacity: Optional[int] = None) -> BCSIndexes:
        """mask: uint8 (or any 1-byte dtype) [H, W] on the GPU.  `capacity` bounds the
        number of index entries kept (default: every block)."""
        job = self._prepare(mask, capacity)
        dev = job['mask'].device
        with torch.cuda.device(dev):
            rc = _lib.load().spx_bcs_index_scheduled(
                _lib.dev_ptr(job['mask']), job['H'], job['W'], self._block_H, self._block_W,
                _lib.dev_ptr(job['row_ptr']), _lib.dev_ptr(job['bcsr']), _lib.dev_ptr(job['col_ptr']),
                _lib.dev_ptr(job['bcsc']), 1 if (self._BCSR and self._BCSC) else 0, _lib.dev_ptr(job['nnz_dev']),
                job['cap'], _lib.dev_ptr(job['row_order']), _lib.dev_ptr(job['col_order']),
                _lib.dev_ptr(job['ws']), job['ws'].numel(), _lib.current_stream(dev))
        _lib.check(rc, 'spx_bcs_index_scheduled')
        return self._wrap(job)

    # ---- values ------------------------------------------------------------------
    def convert(self, dense: torch.Tensor, index: torch.Tensor, block_nnz: int, H: int, W: int,
                idx_kind: int = _lib.IDX_BCSR_I32, nnz_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
        assert dense.shape[-2] == H and dense.shape[-1] == W, \
            f'expected a (..., {H}, {W}) tensor, got {tuple(dense.shape)}'
        lead = tuple(dense.shape[:-2])
        batch = int(np.prod(lead)) if lead else 1
        dense = dense.contiguous()
        out = torch.empty((batch, block_nnz * self._block_size), dtype=dense.dtype, device=dense.device)
        with torch.cuda.device(dense.device):
            rc = _lib.load().spx_bcs_gather(
                _lib.dev_ptr(dense), _lib.dev_ptr(out), _lib.dev_ptr(index), idx_kind, block_nnz,
                _lib.dev_ptr(nnz_dev), batch, H, W, self._block_H, self._block_W, dense.element_size(),
                block_nnz * self._block_size, _lib.current_stream(dense.device))
        _lib.check(rc, 'spx_bcs_gather')
        return out.reshape(lead + (-1,))

    def inverse(self, sparse_val: torch.Tensor, index: torch.Tensor, block_nnz: int, H: int, W: int,
                idx_kind: int = _lib.IDX_BCSR_I32) -> torch.Tensor:
        assert sparse_val.shape[-1] == block_nnz * self._block_size, \
            f'expected (..., {block_nnz * self._block_size}) values, got {tuple(sparse_val.shape)}'
        lead = tuple(sparse_val.shape[:-1])
        batch = int(np.prod(lead)) if lead else 1
        sparse_val = sparse_val.contiguous()
        dense = torch.zeros((batch, H, W), dtype=sparse_val.dtype, device=sparse_val.device)
        with torch.cuda.device(sparse_val.device):
            rc = _lib.load().spx_bcs_scatter(
                _lib.dev_ptr(sparse_val), _lib.dev_ptr(dense), _lib.dev_ptr(index), idx_kind, block_nnz, None,
                batch, H, W, self._block_H, self._block_W, sparse_val.element_size(),
                block_nnz * self._block_size, _lib.current_stream(sparse_val.device))
        _lib.check(rc, 'spx_bcs_scatter')
        return dense.reshape(lead + (H, W))

    def block_sum(self, sparse_val: torch.Tensor, index: torch.Tensor, idx_kind: int, block_nnz: int,
                  H: int, W: int, axis: int) -> torch.Tensor:
        """axis 0: [..., H] sums over W; axis 1: [..., W] sums over H (fp32 accumulate)."""
        lead = tuple(sparse_val.shape[:-1])
        batch = int(np.prod(lead)) if lead else 1
        # values kept at index capacity (dynamic masks) are longer than the live blocks
        stride = sparse_val.shape[-1]
        assert stride >= block_nnz * self._block_size, \
            f'expected at least (..., {block_nnz * self._block_size}) values, got {tuple(sparse_val.shape)}'
        vals = sparse_val.contiguous()
        if vals.dtype not in (torch.float32, torch.float16, torch.bfloat16):
            vals = vals.to(torch.float32)
        n_out = H if axis == 0 else W
        result = torch.empty((batch, n_out), dtype=torch.float32, device=vals.device)
        with torch.cuda.device(vals.device):
            rc = _lib.load().spx_bcs_sum(
                _lib.dev_ptr(vals), _lib.dev_ptr(result), _lib.dev_ptr(index), idx_kind, block_nnz,
                batch, H, W, self._block_H, self._block_W, _lib.dtype_code(vals.dtype), axis,
                stride, _lib.current_stream(vals.device))
        _lib.check(rc, 'spx_bcs_sum')
        return result.to(sparse_val.dtype).reshape(lead + (n_out,))


_bcs_function_cache: Dict[Tuple[int, int, bool, bool], BCSFunctionContext] = {}


def build_indexes_batch(requests) -> List[BCSIndexes]:
    """Indexes of several masks in one library call (spx_bcs_index_batch: the builds that
    qualify share one pair of launches).  `requests` is a sequence of
    (BCSFunctionContext, mask) or (BCSFunctionContext, mask, capacity); all masks on one GPU.
    The results equal those of `context.build_indexes(mask, capacity)` one by one."""
    requests = [tuple(r) + (None,) * (3 - len(r)) for r in requests]
    if not requests:
        return []
    jobs = [ctx._prepare(mask, cap) for ctx, mask, cap in requests]
    dev = jobs[0]['mask'].device
    assert all(j['mask'].device == dev for j in jobs), 'the masks of one batch must be on one device'
    array = (_lib.BcsIndexJob * len(jobs))()
    addr = lambda t: None if t is None else t.data_ptr()
    for slot, (ctx, _, _), job in zip(array, requests, jobs):
        slot.mask = addr(job['mask'])
        slot.H, slot.W, slot.BH, slot.BW = job['H'], job['W'], ctx._block_H, ctx._block_W
        slot.row_ptr, slot.bcsr_idx = addr(job['row_ptr']), addr(job['bcsr'])
        slot.col_ptr, slot.bcsc_idx = addr(job['col_ptr']), addr(job['bcsc'])
        slot.bcsc_i64 = 1 if (ctx._BCSR and ctx._BCSC) else 0
        slot.nnz_dev, slot.cap = addr(job['nnz_dev']), job['cap']
        slot.row_order, slot.col_order = addr(job['row_order']), addr(job['col_order'])
        slot.workspace, slot.workspace_bytes = addr(job['ws']), job['ws'].numel()
    with torch.cuda.device(dev):
        rc = _lib.load().spx_bcs_index_batch(array, len(jobs), _lib.current_stream(dev))
    _lib.check(rc, 'spx_bcs_index_batch')
    return [ctx._wrap(job) for (ctx, _, _), job in zip(requests, jobs)]


def get_bcs_function(block_H: int, block_W: int, BCSR: bool, BCSC: bool) -> BCSFunctionContext:
    """Cached BCSFunctionContext per (block_H, block_W, BCSR, BCSC)."""
    key = (block_H, block_W, bool(BCSR), bool(BCSC))
    ctx = _bcs_function_cache.get(key)
    if ctx is None:
        ctx = _bcs_function_cache[key] = BCSFunctionContext(*key)
    return ctx
