"""Attention over per-batch sequence lengths: batch b attends over its first
`seqlens[b]` positions, the rest of its rows are zero.

Mirrors sparta/specializer/operators/seqlen_dynamic_sparse_attention.py:35-105
(class name, `global_mode`, `set_global_seqlens`, the (B, H, N, E) shapes and its
assertions).  The reference runs three kernels through a [B*H*N*N] fp32 scratch
(`inter_result`, :100-103); here one fused kernel (spx_attention_seqlen_forward)
keeps the scores on chip, so no scratch is held.  Like the reference's extension
the softmax applies no temperature, and there is no backward pass (:27-29).
"""
from typing import Optional

import torch

from sparta_amd import _lib


class SeqlenDynamicSparseAttention(torch.nn.Module):
    r"""Sequence-length sparse attention with dynamic (per call) lengths.

    Args:
        global_mode (bool): all instances share the lengths set through
            :meth:`set_global_seqlens` (sparse pattern set once per batch).

    Shape:
        - Q, K, V: :math:`(B, H, N, E)`; N and E multiples of 32
        - seqlens: int32 :math:`(B,)` on the GPU
        - Output: :math:`(B, H, N, E)`
    """

    global_seqlen: Optional[torch.Tensor] = None

    def __init__(self, global_mode: bool = True):
        super().__init__()
        self.global_mode = global_mode

    @staticmethod
    def set_global_seqlens(seqlens: torch.Tensor):
        """Set the sequence lengths used by every instance in global mode."""
        assert isinstance(seqlens, torch.Tensor)
        assert seqlens.is_cuda
        assert seqlens.dtype == torch.int32, "only support int32 for seqlens"
        SeqlenDynamicSparseAttention.global_seqlen = seqlens

    def forward(self, Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor,
                seqlens: Optional[torch.Tensor] = None) -> torch.Tensor:
        Q, K, V = Q.contiguous(), K.contiguous(), V.contiguous()
        if self.global_mode:
            seqlens = SeqlenDynamicSparseAttention.global_seqlen
        assert seqlens is not None, 'no sequence lengths: pass seqlens or call set_global_seqlens'
        assert seqlens.is_cuda and seqlens.dtype == torch.int32, "only support int32 for seqlens"
        B, H, N, E = Q.shape
        assert K.shape == Q.shape and V.shape == Q.shape and K.dtype == Q.dtype and V.dtype == Q.dtype
        assert B == seqlens.size(0)
        assert N % 32 == 0, 'max sequence length should be divisible by 32'
        assert E % 32 == 0, 'embed dimension size should be divisible by 32'
        out = torch.empty_like(Q)
        rc = _lib.load().spx_attention_seqlen_forward(
            _lib.dtype_code(Q.dtype), _lib.dev_ptr(Q), _lib.dev_ptr(K), _lib.dev_ptr(V), _lib.dev_ptr(out),
            _lib.dev_ptr(seqlens.contiguous()), 1.0, B, H, N, E, 0, _lib.current_stream(Q.device))
        _lib.check(rc, 'spx_attention_seqlen_forward')
        return out
