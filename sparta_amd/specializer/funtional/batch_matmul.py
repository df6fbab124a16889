"""Batched block-sparse matmul: forward kernel plus the two kernels its gradients
need, derived from the forward mode and transposes.

Interface of sparta/specializer/funtional/batch_matmul.py:12-179.
"""
from typing import Any, Dict, List, Optional, Tuple

import torch

from sparta_amd.specializer.kernels import SparTASparseMatMulKernel, OpenAISparseMatMulKernel
from sparta_amd.specializer.funtional.sparse_ctx_base import SparseCtxBase, KernelPlaceholder


def _derive_kernels(mode: str, transpose_A: bool, transpose_B: bool, biased: bool):
    """For C = op(A) op(B): the gradient w.r.t. A and B are matmuls of the other
    two tensors.  Returns, per kernel name, (biased, operand order, transA, transB)
    where the operand order says which of A, B, C plays the role of the new
    kernel's first, second and output tensor."""
    return {
        'forward:C': (biased, 'ABC', transpose_A, transpose_B),
        'backward:A': (False, 'BCA' if transpose_A else 'CBA',
                       transpose_A and transpose_B, transpose_A or not transpose_B),
        'backward:B': (False, 'CAB' if transpose_B else 'ACB',
                       not transpose_A or transpose_B, transpose_A and transpose_B),
    }


def _tile_dims(mode: str, trans_A: bool, trans_B: bool) -> Tuple[str, str]:
    if mode == 'sdd':
        return ('K', 'M') if trans_A else ('M', 'K')
    if mode == 'dsd':
        return ('N', 'K') if trans_B else ('K', 'N')
    return ('M', 'N')


class SparseBatchMatMulCtx(SparseCtxBase):

    def __init__(self, mode: str, transpose_A: bool, transpose_B: bool, biased: bool, compressed: bool):
        super().__init__()
        self._mode = mode
        self._transpose_A = transpose_A
        self._transpose_B = transpose_B
        self._biased = biased
        self._compressed = compressed
        self._activation: Optional[str] = None
        sparse_tensor = 'ABC'[mode.index('s')]
        self._tesa_shapes: Dict[str, Tuple[str, str]] = {}
        for name, (bias, order, tA, tB) in _derive_kernels(mode, transpose_A, transpose_B, biased).items():
            # letter i of the derived mode = sparsity letter of the tensor in role i
            derived_mode = ''.join(mode['ABC'.index(t)] for t in order)
            self._kernels[name] = KernelPlaceholder(
                name=name,
                impls={'sparta': SparTASparseMatMulKernel, 'openai': OpenAISparseMatMulKernel},
                args=dict(mode=derived_mode, biased=bias, transpose_A=tA, transpose_B=tB,
                          compressed=compressed),
                port_map={sparse_tensor: 'ABC'[order.index(sparse_tensor)]},
                connectable=compressed,
            )
            self._tesa_shapes[name] = _tile_dims(derived_mode, tA, tB)
        self._init_sparse_ports([sparse_tensor])

    def set_shape(self, batch_size: int, M: int, K: int, N: int):
        self._kernels['forward:C'].set_shape(batch_size, M, K, N)
        self._kernels['backward:A'].set_shape(*((batch_size, K, N, M) if self._transpose_A
                                                else (batch_size, M, N, K)))
        self._kernels['backward:B'].set_shape(*((batch_size, N, M, K) if self._transpose_B
                                                else (batch_size, K, M, N)))

    def set_activation(self, activation: Optional[str]):
        """Fuse an activation (None or 'relu') into the forward kernel's epilogue; the
        autograd function then masks the incoming gradient with the sign of the output."""
        if activation not in (None, 'relu'):
            raise ValueError(f'unsupported fused activation: {activation!r}')
        if activation is not None and self._mode == 'dds':
            raise ValueError('the fused activation covers the sdd and dsd kernels only')
        self._activation = activation
        fwd = self._kernels['forward:C'].active_kernel()
        if fwd is not None:
            fwd.set_epilogue(activation)

    def build(self, config: Dict[str, Dict[str, Any]]):
        super().build(config)
        fwd = self._kernels['forward:C'].active_kernel()
        if fwd is not None:
            fwd.set_epilogue(self._activation)
            self.forward_C = (lambda A, B, bias: fwd(A, B, bias)) if self._biased else (lambda A, B: fwd(A, B))
            if self._mode == 'dds' and self._compressed:
                kernel = fwd
                self.backward_bias = lambda grad_C: kernel.ports['C'].indexes.sum(grad_C, axis=-2)
            else:
                self.backward_bias = lambda grad_C: grad_C.sum(-2)
        bwd_A = self._kernels['backward:A'].active_kernel()
        if bwd_A is not None:
            if self._transpose_A:
                self.backward_A = lambda grad_C, B: bwd_A(B, grad_C)
            else:
                self.backward_A = lambda grad_C, B: bwd_A(grad_C, B)
        bwd_B = self._kernels['backward:B'].active_kernel()
        if bwd_B is not None:
            if self._transpose_B:
                self.backward_B = lambda grad_C, A: bwd_B(grad_C, A)
            else:
                self.backward_B = lambda grad_C, A: bwd_B(A, grad_C)

    def set_sample_inputs(self, sample_inputs: List[torch.Tensor],
                          sample_grads: Optional[List[torch.Tensor]] = None):
        A, B = sample_inputs[0], sample_inputs[1]
        fwd_inputs = [A, B] + ([sample_inputs[2].detach()] if self._biased else [])
        self._kernels['forward:C'].set_sample_inputs(fwd_inputs)
        if sample_grads is None:
            return
        grad_C = sample_grads[0]
        self._kernels['backward:A'].set_sample_inputs([B, grad_C] if self._transpose_A else [grad_C, B])
        self._kernels['backward:B'].set_sample_inputs([grad_C, A] if self._transpose_B else [A, grad_C])

    def get_connections(self, backward: bool = False):
        """Block dimensions that must agree between kernels sharing a compressed
        tensor: one dict per tile axis, kernel name -> parameter name."""
        if not (self._compressed and backward):
            return []
        return [
            {name: f'BLOCK_SIZE_{dims[axis]}_VALUE' for name, dims in self._tesa_shapes.items()}
            for axis in (0, 1)
        ]

    def dense_forward(self, *args):
        return self._kernels['forward:C'].dense_func(*args)


class SparseBatchMatMulFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx, sparta_ctx: SparseBatchMatMulCtx, input: torch.Tensor, weight: torch.Tensor,
                bias: Optional[torch.Tensor] = None):
        input, weight = input.detach(), weight.detach()
        ctx.sparta_ctx = sparta_ctx
        if bias is None:
            output = sparta_ctx.forward_C(input, weight)
        else:
            output = sparta_ctx.forward_C(input, weight, bias.detach())
        # a fused relu: the gradient passes where the output is positive
        ctx.save_for_backward(input, weight, bias, output if sparta_ctx._activation == 'relu' else None)
        return output

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        input, weight, bias, gate = ctx.saved_tensors
        grad_output = grad_output.detach().contiguous()
        if gate is not None:
            grad_output = grad_output * (gate > 0)
        grad_input = grad_weight = grad_bias = None
        if ctx.needs_input_grad[1]:
            grad_input = ctx.sparta_ctx.backward_A(grad_output, weight)
        if ctx.needs_input_grad[2]:
            grad_weight = ctx.sparta_ctx.backward_B(grad_output, input)
        if bias is not None and ctx.needs_input_grad[3]:
            grad_bias = ctx.sparta_ctx.backward_bias(grad_output)
        return None, grad_input, grad_weight, grad_bias
