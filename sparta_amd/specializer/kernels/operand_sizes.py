"""Element counts the device kernels read and write, and the checks every launch closure
runs against the tensors it is handed before it calls into the library.

The C ABI takes plain pointers: a kernel cannot know how large the allocation behind a
pointer is, and a tensor that is smaller than what the kernel walks is not an exception on
the GPU but a memory fault.  The one way this happens through the Python layer is a
compressed tensor ([batch, nnz * block_H * block_W]) laid out by one index and handed to a
kernel that is bound to another one (other block shape, other mask): the kernel strides the
batch by ITS nnz * block_H * block_W.  Shape asserts of the reference's operators that these
checks correspond to: sparta/specializer/operators/sparse_softmax.py:57-71,
sparse_attention.py:98-108.  All checks raise AssertionError (what the tuner treats as an
invalid trial) and need no GPU: they only look at `numel()`.
"""
from typing import NamedTuple, Optional

import torch


def require_numel(what: str, name: str, tensor: Optional[torch.Tensor], numel: int):
    """The kernel `what` reads or writes exactly `numel` elements behind `name`."""
    assert tensor is not None, f'{what}: {name} is required'
    assert tensor.numel() == numel, (
        f'{what}: {name} has {tensor.numel()} elements (shape {tuple(tensor.shape)}), '
        f'the kernel is bound to {numel}')


class MatmulExtent(NamedTuple):
    """What one bound spx_matmul closure reads (A, B, bias) and writes (C), in elements."""
    A: int
    B: int
    bias: int
    C: int


def matmul_extent(mode: str, compressed: bool, batch: int, M: int, K: int, N: int,
                  sparse_stride: int) -> MatmulExtent:
    """`sparse_stride` = (live blocks, or index capacity for a port kept at capacity) x
    elements per block of the index the kernel is bound to."""
    dense = {'A': batch * M * K, 'B': batch * K * N, 'C': batch * M * N}
    if compressed:
        dense[{'sdd': 'A', 'dsd': 'B', 'dds': 'C'}[mode]] = batch * sparse_stride
    return MatmulExtent(dense['A'], dense['B'], batch * N, dense['C'])


def check_matmul_operands(extent: MatmulExtent, A: torch.Tensor, B: torch.Tensor,
                          bias: Optional[torch.Tensor], biased: bool):
    require_numel('spx_matmul', 'A', A, extent.A)
    require_numel('spx_matmul', 'B', B, extent.B)
    if biased:
        require_numel('spx_matmul', 'bias', bias, extent.bias)


def softmax_extent(compressed: bool, batch: int, H: int, W: int, sparse_stride: int) -> int:
    """Elements of x, y and the gradients of one bound softmax closure."""
    return batch * (sparse_stride if compressed else H * W)


class AttentionExtent(NamedTuple):
    """Elements behind the pointers of the fused attention kernels."""
    q: int          # query, output, their gradients
    kv: int         # key, value, their gradients
    rows: int       # one float per query (log-sum-exp, row constants)
    probs: int      # compressed probabilities / score gradients


def attention_extent(batch: int, Nt: int, Ns: int, E: int, nnz: int, BH: int, BW: int) -> AttentionExtent:
    return AttentionExtent(batch * Nt * E, batch * Ns * E, batch * Nt, batch * nnz * BH * BW)


def check_index_matches(what: str, indexes, Nt: int, Ns: int):
    """The index a fused attention kernel walks must describe an Nt x Ns mask."""
    assert (indexes.H, indexes.W) == (Nt, Ns), \
        f'{what}: the index covers a {indexes.H} x {indexes.W} mask, the operands are {Nt} x {Ns}'
