"""Sparse batched matmul operator C = op(A) op(B) with a mask on A, B or C
(interface of sparta/specializer/operators/sparse_matmul.py:12-136)."""
from typing import Optional

import torch

from sparta_amd.specializer.operators.operator_base import OperatorBase
from sparta_amd.specializer.funtional import SparseBatchMatMulCtx, SparseBatchMatMulFunc


class SparseBatchMatMul(OperatorBase):
    r"""Args:
        A_mask / B_mask / C_mask: exactly one 2-D mask; selects the 'sdd' / 'dsd' /
            'dds' kernel family.
        transpose_A: A is stored (B, K, M) instead of (B, M, K).
        transpose_B: B is stored (B, N, K) instead of (B, K, N).
        compressed: the masked tensor is exchanged in block-compressed form
            (B, nnz * block_h * block_w) instead of dense.

    Example::

        mask = sparta_amd.testing.block_mask((1024, 1024), block=(32, 32), sparsity=0.9)
        matmul = sparta_amd.nn.SparseBatchMatMul(C_mask=mask)
        sparta_amd.nn.tune(matmul, sample_inputs=[
            torch.rand((4, 1024, 1024), device='cuda'), torch.rand((4, 1024, 1024), device='cuda')])
    """

    __sparse_func__ = SparseBatchMatMulFunc

    def __init__(self, A_mask: Optional[torch.Tensor] = None, B_mask: Optional[torch.Tensor] = None,
                 C_mask: Optional[torch.Tensor] = None, transpose_A: bool = False,
                 transpose_B: bool = False, compressed: bool = True):
        super().__init__()
        self._transpose_A = transpose_A
        self._transpose_B = transpose_B
        M = K = N = None
        if A_mask is not None:
            mode = 'sdd'
            K, M = A_mask.shape if transpose_A else A_mask.shape[::-1]
        elif B_mask is not None:
            mode = 'dsd'
            N, K = B_mask.shape if transpose_B else B_mask.shape[::-1]
        elif C_mask is not None:
            mode = 'dds'
            M, N = C_mask.shape
        else:
            raise ValueError('expected a sparse mask on A / B / C')
        self._sparse_ctx = SparseBatchMatMulCtx(mode=mode, transpose_A=transpose_A, transpose_B=transpose_B,
                                                biased=False, compressed=compressed)
        self._shape = {'batch_size': None, 'M': M, 'K': K, 'N': N}
        self.update_mask(A_mask, B_mask, C_mask)

    def update_mask(self, A_mask: Optional[torch.Tensor] = None, B_mask: Optional[torch.Tensor] = None,
                    C_mask: Optional[torch.Tensor] = None):
        given = {p: m for p, m in (('A', A_mask), ('B', B_mask), ('C', C_mask)) if m is not None}
        if len(given) > 1:
            raise ValueError('linear operators with multiple sparse masks are not supported')
        if not given:
            raise ValueError('expected a sparse mask on A / B / C')
        self._set_mask(given)

    def _read_sample_inputs(self, A: torch.Tensor, B: torch.Tensor):
        batch_size = A.shape[0]
        K, M = A.shape[1:] if self._transpose_A else A.shape[:0:-1]
        N, K2 = B.shape[1:] if self._transpose_B else B.shape[:0:-1]
        assert K == K2 and B.shape[0] == batch_size, \
            f'incompatible operand shapes {tuple(A.shape)} and {tuple(B.shape)}'
        self._shape = {'batch_size': batch_size, 'M': M, 'K': K, 'N': N}
