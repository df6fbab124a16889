"""Sparse attention operator softmax_masked(Q K^T / sqrt(E)) V
(interface of sparta/specializer/operators/sparse_attention.py:14-238).

It is assembled from three sparse operators that share one BCSR index and one
compressed layout: a sparse-output matmul for Q K^T, the masked softmax, and a
sparse-input matmul for P V.  When no gradient is required the forward pass runs
the fused kernel instead (spx_attention_forward), which keeps the scores in
registers / LDS and never writes them to HBM.
"""
import warnings
from typing import Any, Dict, List, Optional

import numpy as np
import torch

from sparta_amd import _lib
from sparta_amd.specializer.operators.operator_base import OperatorBase
from sparta_amd.specializer.operators.sparse_matmul import SparseBatchMatMul
from sparta_amd.specializer.operators.sparse_softmax import SparseSoftmax
from sparta_amd.specializer.kernels import KernelBase, PortConfig
from sparta_amd.specializer.funtional.sparse_ctx_base import check_shared_block_shapes
from sparta_amd.specializer.kernels.operand_sizes import attention_extent, check_index_matches, require_numel

# operator-level name -> (attribute, sparse port of that operator)
_PARTS = (('qk', '_matmul_qk', 'C'), ('sm', '_softmax', 'y'), ('out', '_matmul_out', 'A'))


class _FusedAttentionFunc(torch.autograd.Function):
    """Forward: one launch gives the output and the probabilities.  Backward: a row-side
    launch for the query gradient and a column-side launch for the key and value gradients,
    both reading the saved probabilities (block shapes the column-side kernel does not
    cover take the two transposed sparse x dense products of the matmul operators)."""

    @staticmethod
    def forward(ctx, op: 'SparseAttention', query: torch.Tensor, key: torch.Tensor, value: torch.Tensor):
        q, k, v = query.detach(), key.detach(), value.detach()
        # the index of this forward pass: the probabilities are laid out by it, and a mask update
        # between forward and backward must not change what the backward kernels walk
        ctx.indexes = op._sparse_port.indexes
        out, probs = op._fused_forward_train(q, k, v)
        ctx.save_for_backward(q, k, v, out, probs)
        ctx.op = op
        return out

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        q, k, v, out, probs = ctx.saved_tensors
        op = ctx.op
        out_ctx, qk_ctx = op._matmul_out._sparse_ctx, op._matmul_qk._sparse_ctx
        grad_out = grad_out.detach().contiguous()
        need_q, need_k, need_v = ctx.needs_input_grad[1:4]
        grad_q = grad_k = grad_v = None
        indexes = ctx.indexes
        if (need_k or need_v) and op._fused_backward_kv_supported(grad_out, indexes):
            # two launches: the row side gives grad_q and the row constants, the column side
            # recomputes the score gradient from the probabilities for grad_k and grad_v
            _, grad_q, row_dot = op._fused_backward_scores(grad_out, out, probs, k, v, store_scores=False,
                                                           indexes=indexes)
            grad_k, grad_v = op._fused_backward_kv(grad_out, q, v, probs, row_dot, indexes)
        else:
            # the operator kernels are bound to the operator's current index
            assert indexes is op._sparse_port.indexes, \
                'the mask was updated between forward and backward of a SparseAttention call'
            if need_v:
                grad_v = out_ctx.backward_B(grad_out, probs)
            if need_q or need_k:
                grad_scores, grad_q, _ = op._fused_backward_scores(grad_out, out, probs, k, v, store_scores=need_k,
                                                                   indexes=indexes)
                if need_k:
                    grad_k = qk_ctx.backward_B(grad_scores, q)
        return None, grad_q if need_q else None, grad_k if need_k else None, grad_v if need_v else None


class _RecomputeAttentionFunc(torch.autograd.Function):
    """Training path that keeps no probabilities: the forward kernel records one number per
    query (the log-sum-exp of its score row), and the row-side and column-side backward
    kernels recompute the probabilities of every live block from q, k and that number."""

    @staticmethod
    def forward(ctx, op: 'SparseAttention', query: torch.Tensor, key: torch.Tensor, value: torch.Tensor):
        q, k, v = query.detach().contiguous(), key.detach().contiguous(), value.detach().contiguous()
        # the index of this forward pass: the log-sum-exp belongs to its set of live blocks, so
        # the backward kernels walk the same index even if the mask has been updated since
        ctx.indexes = op._sparse_port.indexes
        out, row_lse = op._fused_forward_lse(q, k, v)
        ctx.save_for_backward(q, k, v, out, row_lse)
        ctx.op = op
        return out

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        q, k, v, out, row_lse = ctx.saved_tensors
        op = ctx.op
        grad_out = grad_out.detach().contiguous()
        need_q, need_k, need_v = ctx.needs_input_grad[1:4]
        grad_q, row_dot = op._recompute_backward_q(grad_out, out, q, k, v, row_lse, ctx.indexes)
        grad_k = grad_v = None
        if need_k or need_v:
            grad_k, grad_v = op._recompute_backward_kv(grad_out, q, k, v, row_lse, row_dot, ctx.indexes)
        return None, grad_q if need_q else None, grad_k if need_k else None, grad_v if need_v else None


class SparseAttention(OperatorBase):
    r"""Args:
        mask: (N_target, N_source) mask of the score entries that take part.
        fused: run the single fused forward kernel when autograd is not recording
            (default True).  The three-operator pipeline is always built as well and
            is used whenever gradients are needed.
        recompute: with a mask that is uniform inside its blocks, train without storing
            the probabilities (default True): the backward kernels recompute them from
            q, k and one number per query.  Masks with partly live blocks, and
            `recompute=False`, keep the probabilities of the live blocks for the backward pass.
        fused_tile_cfg: tile configuration of the fused kernel (0 = the library's choice;
            see spx_tile_cfg_info for the others).

    Shape: query (B*H, N_target, E), key / value (B*H, N_source, E) -> (B*H, N_target, E).
    """

    def __init__(self, mask: torch.Tensor, fused: bool = True, fused_tile_cfg: int = 0, recompute: bool = True):
        super().__init__()
        self._recompute = recompute
        self.mask = mask
        self._Nt, self._Ns = mask.shape
        self._matmul_qk = SparseBatchMatMul(C_mask=mask, transpose_A=False, transpose_B=True, compressed=True)
        self._softmax = SparseSoftmax(mask=mask, compressed=True)
        self._matmul_out = SparseBatchMatMul(A_mask=mask, transpose_A=False, transpose_B=False, compressed=True)
        self._sparse_port: Optional[PortConfig] = None
        self._fused = fused
        self._fused_tile_cfg = int(fused_tile_cfg)
        self._fused_mask_key = None   # index object the cached element mask belongs to
        self._fused_mask = None
        self._inv_temperature = 1.0
        self._warned_unfused = False
        self._tile_strict = False   # True while tune_tile_config times a variant: a refusal must show
        self.ready = False

    def _parts(self):
        return [(name, getattr(self, attr), port) for name, attr, port in _PARTS]

    # ---- forward ---------------------------------------------------------------------
    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor):
        if self.ready and self._fused and self._fused_supported(query):
            recording = torch.is_grad_enabled() and (query.requires_grad or key.requires_grad or value.requires_grad)
            if not recording:
                return self._fused_forward(query, key, value)
            if self._recompute and self._recompute_supported(query):
                return _RecomputeAttentionFunc.apply(self, query, key, value)
            if self._fused_train_supported(query):
                return _FusedAttentionFunc.apply(self, query, key, value)
        if self.ready and self._fused and not self._warned_unfused and torch.is_grad_enabled() and (
                query.requires_grad or key.requires_grad or value.requires_grad):
            self._warned_unfused = True
            indexes = self._sparse_port.indexes
            ctxs = (self._matmul_qk._sparse_ctx, self._matmul_out._sparse_ctx)
            if all(hasattr(c, 'backward_B') for c in ctxs):
                why = (f'no fused training kernel for {query.dtype} inputs of head dim {query.shape[-1]} with '
                       f'{indexes.block_H}x{indexes.block_W} score blocks (16-bit types, head dims 64 / 128 and '
                       'blocks of 32 / 64 / 128 are covered)')
            else:
                why = 'the backward kernels of the operator were not built (no backward:* entries in its configuration)'
            warnings.warn(f'SparseAttention: {why}; this step runs as three forward launches and six backward launches')
        scores = self._matmul_qk.forward(query, key)
        probs = self._softmax.forward(scores)
        return self._matmul_out.forward(probs, value)

    def _fused_train_supported(self, query: torch.Tensor) -> bool:
        """The training forward kernel (output and probabilities in one launch) needs the
        block shapes it covers, 3-D inputs and the matmul operators' backward kernels built."""
        indexes = self._sparse_port.indexes
        BH, BW, E = indexes.block_H, indexes.block_W, query.shape[-1]
        if not (query.dim() == 3 and BH in (32, 64, 128) and BW in (32, 64, 128) and E in (64, 128) and BW * E // 8 >= BH * 4):
            return False
        ctxs = (self._matmul_qk._sparse_ctx, self._matmul_out._sparse_ctx)
        return all(hasattr(c, 'backward_B') for c in ctxs)

    def _recompute_supported(self, query: torch.Tensor) -> bool:
        """The kernels that recompute the probabilities cover block-level masks, 3-D 16-bit
        inputs and the block shapes of both backward kernels, and walk both indexes."""
        indexes = self._sparse_port.indexes
        BH, BW, E = indexes.block_H, indexes.block_W, query.shape[-1]
        return (query.dim() == 3 and BH in (32, 64, 128) and BW in (32, 64, 128) and E in (64, 128)
                and BW * E // 8 >= BH * 4 and BH * E >= 32 * BW and BH <= 2 * BW
                and getattr(indexes, 'col_ptr', None) is not None and getattr(indexes, 'row_ptr', None) is not None
                and self._element_mask() is None)

    def _check_operands(self, what: str, indexes, batch: int, E: int, q_like=(), kv_like=(), rows=(),
                        probs=(), nnz=None):
        """Sizes of the tensors behind the pointers of one fused-kernel call, against what the
        kernel walks for `batch` entries of the index's mask; AssertionError before any launch."""
        check_index_matches(what, indexes, self._Nt, self._Ns)
        want = attention_extent(batch, self._Nt, self._Ns, E, indexes.block_nnz if nnz is None else nnz,
                                indexes.block_H, indexes.block_W)
        for group, numel in ((q_like, want.q), (kv_like, want.kv), (rows, want.rows), (probs, want.probs)):
            for name, tensor in group:
                if tensor is not None:
                    require_numel(what, name, tensor, numel)

    def _fused_forward_lse(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
        """(output, log-sum-exp per query) from spx_attention_forward_lse."""
        indexes = self._sparse_port.indexes
        batch, _, E = q.shape
        out = torch.empty_like(q)
        row_lse = torch.empty((batch, self._Nt), dtype=torch.float32, device=q.device)
        self._check_operands('spx_attention_forward_lse', indexes, batch, E, q_like=[('q', q)],
                             kv_like=[('k', k), ('v', v)], nnz=0)
        rc = _lib.load().spx_attention_forward_lse(
            _lib.dtype_code(q.dtype), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v), _lib.dev_ptr(out),
            _lib.dev_ptr(row_lse), _lib.dev_ptr(indexes.row_ptr), _lib.dev_ptr(indexes._bcsr_buf), None,
            float(self._inv_temperature), batch, self._Nt, self._Ns, E, indexes.block_H, indexes.block_W,
            _lib.current_stream(q.device))
        _lib.check(rc, 'spx_attention_forward_lse')
        return out, row_lse

    def _recompute_backward_q(self, grad_out, out, q, k, v, row_lse, indexes=None):
        """(query gradient, row constants) from spx_attention_backward_q."""
        indexes = self._sparse_port.indexes if indexes is None else indexes
        batch, _, E = grad_out.shape
        grad_q = torch.empty_like(q)
        row_dot = torch.empty((batch, self._Nt), dtype=torch.float32, device=q.device)
        self._check_operands('spx_attention_backward_q', indexes, batch, E,
                             q_like=[('grad_out', grad_out), ('out', out), ('q', q)],
                             kv_like=[('k', k), ('v', v)], rows=[('row_lse', row_lse)], nnz=0)
        rc = _lib.load().spx_attention_backward_q(
            _lib.dtype_code(q.dtype), _lib.dev_ptr(grad_out), _lib.dev_ptr(out), _lib.dev_ptr(q), _lib.dev_ptr(k),
            _lib.dev_ptr(v), _lib.dev_ptr(row_lse), _lib.dev_ptr(grad_q), _lib.dev_ptr(row_dot),
            _lib.dev_ptr(indexes.row_ptr), _lib.dev_ptr(indexes._bcsr_buf), float(self._inv_temperature),
            batch, self._Nt, self._Ns, E, indexes.block_H, indexes.block_W, _lib.current_stream(q.device))
        _lib.check(rc, 'spx_attention_backward_q')
        return grad_q, row_dot

    def _recompute_backward_kv(self, grad_out, q, k, v, row_lse, row_dot, indexes=None):
        """(key gradient, value gradient) from spx_attention_backward_kv_recompute."""
        indexes = self._sparse_port.indexes if indexes is None else indexes
        batch, _, E = grad_out.shape
        grad_k = torch.empty_like(k)
        grad_v = torch.empty_like(v)
        idx = indexes._bcsc_buf
        kind = _lib.IDX_BCSC_I64 if idx.dtype == torch.int64 else _lib.IDX_BCSC_I32
        self._check_operands('spx_attention_backward_kv_recompute', indexes, batch, E,
                             q_like=[('grad_out', grad_out), ('q', q)], kv_like=[('k', k), ('v', v)],
                             rows=[('row_lse', row_lse), ('row_dot', row_dot)], nnz=0)
        rc = _lib.load().spx_attention_backward_kv_recompute(
            _lib.dtype_code(q.dtype), _lib.dev_ptr(grad_out), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v),
            _lib.dev_ptr(row_lse), _lib.dev_ptr(row_dot), _lib.dev_ptr(grad_k), _lib.dev_ptr(grad_v),
            _lib.dev_ptr(indexes.col_ptr), _lib.dev_ptr(idx), kind, float(self._inv_temperature),
            batch, self._Nt, self._Ns, E, indexes.block_H, indexes.block_W, _lib.current_stream(q.device))
        _lib.check(rc, 'spx_attention_backward_kv_recompute')
        return grad_k, grad_v

    def _element_mask(self):
        indexes = self._sparse_port.indexes
        if self._fused_mask_key is not indexes:
            # A mask that is uniform inside its blocks needs no per-element test in the
            # kernel; decided once per index build (one synchronising comparison).
            block_level = indexes.is_block_uniform()
            self._fused_mask = None if block_level else indexes.raw_mask
            self._fused_mask_key = indexes
        return self._fused_mask

    def _fused_forward_train(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor):
        """(output, compressed probabilities) from spx_attention_forward_train."""
        indexes = self._sparse_port.indexes
        mask = self._element_mask()
        batch, _, E = query.shape
        q, k, v = query.contiguous(), key.contiguous(), value.contiguous()
        out = torch.empty_like(q)
        probs = torch.empty((batch, indexes.block_nnz * indexes.block_H * indexes.block_W), dtype=q.dtype, device=q.device)
        self._check_operands('spx_attention_forward_train', indexes, batch, E, q_like=[('q', q)],
                             kv_like=[('k', k), ('v', v)])
        rc = _lib.load().spx_attention_forward_train(
            _lib.dtype_code(q.dtype), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v), _lib.dev_ptr(out),
            _lib.dev_ptr(probs), probs.shape[1], _lib.dev_ptr(indexes.row_ptr), _lib.dev_ptr(indexes._bcsr_buf),
            _lib.dev_ptr(mask), float(self._inv_temperature), batch, self._Nt, self._Ns, E,
            indexes.block_H, indexes.block_W, _lib.current_stream(q.device))
        _lib.check(rc, 'spx_attention_forward_train')
        return out, probs

    def _fused_backward_scores(self, grad_out, out, probs, key, value, store_scores=True, indexes=None):
        """(compressed score gradient or None, query gradient, row constants) from
        spx_attention_backward_scores."""
        indexes = self._sparse_port.indexes if indexes is None else indexes
        batch, _, E = grad_out.shape
        k, v = key.contiguous(), value.contiguous()
        grad_scores = torch.empty_like(probs) if store_scores else None
        grad_q = torch.empty_like(grad_out)
        row_dot = torch.empty((batch, self._Nt), dtype=torch.float32, device=grad_out.device)
        self._check_operands('spx_attention_backward_scores', indexes, batch, E,
                             q_like=[('grad_out', grad_out), ('out', out)], kv_like=[('k', k), ('v', v)],
                             probs=[('probs', probs)])
        rc = _lib.load().spx_attention_backward_scores(
            _lib.dtype_code(grad_out.dtype), _lib.dev_ptr(grad_out), _lib.dev_ptr(out), _lib.dev_ptr(probs),
            _lib.dev_ptr(k), _lib.dev_ptr(v), _lib.dev_ptr(grad_scores), _lib.dev_ptr(grad_q), _lib.dev_ptr(row_dot),
            probs.shape[1], _lib.dev_ptr(indexes.row_ptr), _lib.dev_ptr(indexes._bcsr_buf),
            float(self._inv_temperature), batch, self._Nt, self._Ns, E, indexes.block_H, indexes.block_W,
            _lib.current_stream(grad_out.device))
        _lib.check(rc, 'spx_attention_backward_scores')
        return grad_scores, grad_q, row_dot

    def _fused_backward_kv_supported(self, grad_out: torch.Tensor, indexes=None) -> bool:
        """The column-side kernel needs the BCSC index next to the BCSR one (the probabilities
        are stored in BCSR order) and the block shapes it covers."""
        indexes = self._sparse_port.indexes if indexes is None else indexes
        BH, BW, E = indexes.block_H, indexes.block_W, grad_out.shape[-1]
        return (getattr(indexes, 'col_ptr', None) is not None and getattr(indexes, 'row_ptr', None) is not None
                and BH in (32, 64, 128) and BW in (32, 64, 128) and E in (64, 128) and BH * E >= 32 * BW)

    def _fused_backward_kv(self, grad_out, query, value, probs, row_dot, indexes=None):
        """(key gradient, value gradient) from spx_attention_backward_kv."""
        indexes = self._sparse_port.indexes if indexes is None else indexes
        batch, _, E = grad_out.shape
        q, v = query.contiguous(), value.contiguous()
        grad_k = torch.empty_like(v)
        grad_v = torch.empty_like(v)
        idx = indexes._bcsc_buf
        kind = _lib.IDX_BCSC_I64 if idx.dtype == torch.int64 else _lib.IDX_BCSC_I32
        self._check_operands('spx_attention_backward_kv', indexes, batch, E,
                             q_like=[('grad_out', grad_out), ('q', q)], kv_like=[('v', v)],
                             rows=[('row_dot', row_dot)], probs=[('probs', probs)])
        rc = _lib.load().spx_attention_backward_kv(
            _lib.dtype_code(grad_out.dtype), _lib.dev_ptr(grad_out), _lib.dev_ptr(q), _lib.dev_ptr(v),
            _lib.dev_ptr(probs), _lib.dev_ptr(row_dot), _lib.dev_ptr(grad_k), _lib.dev_ptr(grad_v), probs.shape[1],
            _lib.dev_ptr(indexes.col_ptr), _lib.dev_ptr(idx), kind, float(self._inv_temperature),
            batch, self._Nt, self._Ns, E, indexes.block_H, indexes.block_W, _lib.current_stream(grad_out.device))
        _lib.check(rc, 'spx_attention_backward_kv')
        return grad_k, grad_v

    def _fused_supported(self, query: torch.Tensor) -> bool:
        """The fused kernel covers 16-bit inputs, head dims 32 / 64 / 128 and score
        blocks of 16..128; everything else takes the three-operator pipeline."""
        indexes = self._sparse_port.indexes
        return (query.dtype in (torch.float16, torch.bfloat16) and query.shape[-1] in (32, 64, 128)
                and indexes.block_H in (16, 32, 64, 128) and indexes.block_W in (16, 32, 64, 128))

    def _fused_forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor):
        indexes = self._sparse_port.indexes
        self._element_mask()
        lead = query.shape[:-2]
        E = query.shape[-1]
        batch = int(np.prod(lead)) if len(lead) else 1
        q, k, v = query.contiguous(), key.contiguous(), value.contiguous()
        out = torch.empty_like(q)
        self._check_operands('spx_attention_forward', indexes, batch, E, q_like=[('q', q)],
                             kv_like=[('k', k), ('v', v)], nnz=0)
        while True:
            rc = _lib.load().spx_attention_forward(
                _lib.dtype_code(q.dtype), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v), _lib.dev_ptr(out),
                _lib.dev_ptr(indexes.row_ptr), _lib.dev_ptr(indexes._bcsr_buf), _lib.dev_ptr(self._fused_mask),
                float(self._inv_temperature), batch, self._Nt, self._Ns, E,
                indexes.block_H, indexes.block_W, self._fused_tile_cfg, _lib.current_stream(q.device))
            if rc == _lib.E_CONFIG and self._fused_tile_cfg and not self._tile_strict:
                self._fused_tile_cfg = 0   # a tuned variant that does not take these shapes: the library's choice
                continue
            break
        _lib.check(rc, 'spx_attention_forward')
        return out

    # ---- masks -----------------------------------------------------------------------
    def update_mask(self, mask: torch.Tensor):
        self.mask = mask
        if self.ready:
            self._sparse_port.set_mask(mask)
            for _, op, _ in self._parts():
                op._sparse_ctx.update_func()
        else:
            for _, op, _ in self._parts():
                for ports in op._sparse_ctx.sparse_ports.values():
                    for port in ports:
                        port.set_mask(mask)

    # ---- build -----------------------------------------------------------------------
    def _check_qkv(self, query, key, value):
        qB, kB, vB = (int(np.prod(t.shape[:-2])) for t in (query, key, value))
        (qN, qE), (kN, kE), (vN, vE) = (t.shape[-2:] for t in (query, key, value))
        assert qB == kB == vB, 'query, key and value should have the same batch size'
        assert qN == self._Nt, f'expect query shape (?, {self._Nt}, ?), got {tuple(query.shape)}'
        assert kN == self._Ns, f'expect key shape (?, {self._Ns}, ?), got {tuple(key.shape)}'
        assert vN == self._Ns, f'expect value shape (?, {self._Ns}, ?), got {tuple(value.shape)}'
        assert qE == kE == vE, 'query, key and value should have the same embed dim'
        return qE

    def _set_temperature(self, E: int):
        self._softmax.set_temperature(np.sqrt(E))
        self._inv_temperature = 1.0 / float(np.sqrt(E))

    def build(self, config: Dict[str, Any], sample_inputs: List[torch.Tensor]):
        query, key, value = sample_inputs
        self._set_temperature(self._check_qkv(query, key, value))
        # The parts only read the shapes of their sample inputs: the dense score tensor
        # (batch x N_target x N_source) is never materialised.
        scores = torch.empty(tuple(query.shape[:-1]) + (self._Ns,), dtype=query.dtype, device='meta')
        part_inputs = {'qk': [query, key], 'sm': [scores], 'out': [scores, value]}

        # One port (hence one index and one compressed layout) for every selected kernel.
        shared: Optional[PortConfig] = None
        for name, op, op_port in self._parts():
            for kernel_name, placeholder in op._sparse_ctx.get_kernel_placeholders().items():
                kernel: KernelBase = placeholder.possible_kernels[config[f'{name}/{kernel_name}']['_impl']]
                kernel_port = placeholder.port_map[op_port]
                if shared is None:
                    shared = kernel.ports[kernel_port]
                else:
                    shared.connect(kernel, kernel_port)
        self._sparse_port = shared

        for name, op, _ in self._parts():
            prefix = f'{name}/'
            op.build(config={k[len(prefix):]: v for k, v in config.items() if k.startswith(prefix)},
                     sample_inputs=part_inputs[name])
        # the three parts share one index: a part built later must not have changed the block
        # shape under a part built before it
        for name, op, _ in self._parts():
            prefix = f'{name}/'
            check_shared_block_shapes(op._sparse_ctx._kernels, {k[len(prefix):] for k in config if k.startswith(prefix)})
        if 'fused/forward' in config:   # written by tune(..., tile_configs=...)
            self._fused_tile_cfg = int(config['fused/forward'].get('TILE_CFG', 0) or 0)
        self.ready = True

    def tune_tile_config(self, sample_inputs: List[torch.Tensor], num_warmups: int = 10, num_iters: int = 10):
        """Time the fused forward kernel under every tile configuration of the library's
        attention table on `sample_inputs` (device time), keep the fastest one whose output
        agrees with the three-operator pipeline, and return it as a configuration entry
        ({'fused/forward': {'TILE_CFG': id}}, accepted by build()); None when the fused kernel
        does not take these inputs.  The operator must be built."""
        from sparta_amd.testing import profile
        query, key, value = (t.detach() for t in sample_inputs)
        if not (self.ready and self._fused and self._fused_supported(query)):
            return None
        with torch.no_grad():
            scores = self._matmul_qk.forward(query, key)
            want = self._matmul_out.forward(self._softmax.forward(scores), value)
            del scores
            best_id, best_latency = 0, float('inf')
            self._tile_strict = True
            try:
                for tile in _lib.tile_configs(_lib.OP_ATTENTION):
                    self._fused_tile_cfg = tile['id']
                    try:
                        latency = profile(self._fused_forward, [query, key, value], [want], num_warmups, num_iters, cuda=True)
                    except AssertionError:   # the configuration does not take this block shape / head dim
                        latency = float('inf')
                    if latency < best_latency:
                        best_id, best_latency = tile['id'], latency
            finally:
                self._tile_strict = False
        self._fused_tile_cfg = best_id
        return {'fused/forward': {'TILE_CFG': best_id}}

    def set_sample_inputs(self, sample_inputs: List[torch.Tensor],
                          sample_grads: Optional[List[torch.Tensor]] = None):
        query, key, value = sample_inputs
        self._set_temperature(query.shape[-1])
        need_grad = sample_grads is not None
        if need_grad:
            query, key, value = (t.detach().requires_grad_(True) for t in (query, key, value))
        with warnings.catch_warnings():
            warnings.simplefilter('ignore')
            scores = self._matmul_qk.forward(query, key)
            probs = self._softmax.forward(scores)
            grad_scores = grad_probs = None
            if need_grad:
                scores.retain_grad()
                probs.retain_grad()
                self._matmul_out.forward(probs, value).backward(sample_grads[0])
                grad_scores, grad_probs = [scores.grad], [probs.grad]
                query, key, value = query.detach(), key.detach(), value.detach()
        self._matmul_qk.set_sample_inputs([query, key], grad_scores)
        self._softmax.set_sample_inputs([scores], grad_probs)
        self._matmul_out.set_sample_inputs([probs, value], sample_grads)

    # ---- tuning support ----------------------------------------------------------------
    @staticmethod
    def _prefixed(parts: Dict[str, Dict[str, Any]], backward: bool):
        return {
            f'{name}/{kernel}': value
            for name in ('qk', 'sm', 'out')
            for kernel, value in parts[name].items()
            if backward or kernel.startswith('forward')
        }

    def get_search_space(self, backward: bool = False):
        return self._prefixed({name: op.get_search_space(backward=True) for name, op, _ in self._parts()},
                              backward)

    def get_connections(self, backward: bool = False):
        """The block shape of the score matrix is shared by all three operators,
        whether or not backward kernels are tuned."""
        per_op = [op.get_connections(backward=True) for _, op, _ in self._parts()]
        return [
            self._prefixed(dict(zip(('qk', 'sm', 'out'), axis)), backward)
            for axis in zip(*per_op)
        ]

    def get_kernel_placeholders(self, backward: bool = False):
        return self._prefixed({name: op.get_kernel_placeholders(backward=True) for name, op, _ in self._parts()},
                              backward)
