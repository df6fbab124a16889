"""Batched masked block-sparse softmax context and autograd function.

Interface of sparta/specializer/funtional/batch_softmax.py:13-103.
"""
from typing import Any, Dict, List, Optional

import numpy as np
import torch

from sparta_amd.specializer.kernels import (
    SparTASparseSoftmaxForwardKernel, SparTASparseSoftmaxBackwardKernel,
)
from sparta_amd.specializer.funtional.sparse_ctx_base import SparseCtxBase, KernelPlaceholder

_SHARED_DIMS = ('BLOCK_SIZE_H_VALUE', 'BLOCK_SIZE_W_VALUE')


class SparseBatchSoftmaxCtx(SparseCtxBase):

    def __init__(self, compressed: bool, temperature: float = 1):
        super().__init__()
        self._compressed = compressed
        self._batch_size: Optional[int] = None
        self.set_temperature(temperature)
        for name, cls in (('forward:y', SparTASparseSoftmaxForwardKernel),
                          ('backward:x', SparTASparseSoftmaxBackwardKernel)):
            self._kernels[name] = KernelPlaceholder(
                name=name, impls={'sparta': cls}, args={'compressed': compressed},
                port_map={'y': 'y'}, connectable=compressed)
        self._init_sparse_ports(['y'])

    def set_temperature(self, temperature: float):
        # kernels multiply by the inverse temperature
        self._T = np.float32(1 / temperature)

    def set_shape(self, batch_size: int, H: int, W: int):
        for kernel in self._kernels.values():
            kernel.set_shape(batch_size, H, W)
        self._batch_size = batch_size

    def build(self, config: Dict[str, Dict[str, Any]]):
        super().build(config)
        fwd = self._kernels['forward:y'].active_kernel()
        if fwd is not None:
            self.forward = lambda x: fwd(x, self._T)
        bwd = self._kernels['backward:x'].active_kernel()
        if bwd is not None:
            self.backward = lambda grad, output: bwd(grad, output, self._T)

    def set_sample_inputs(self, sample_inputs: List[torch.Tensor],
                          sample_grads: Optional[List[torch.Tensor]] = None):
        x = sample_inputs[0]
        self._kernels['forward:y'].set_sample_inputs([x, self._T])
        if sample_grads is not None:
            y = self._kernels['forward:y'].dense_func(x, self._T)
            self._kernels['backward:x'].set_sample_inputs([sample_grads[0], y, self._T])

    def get_conditions(self, impls: Dict[str, str]):
        if self._compressed and len(impls) > 1:
            return [[f'forward:y;{dim}', f'backward:x;{dim}'] for dim in _SHARED_DIMS]
        return []

    def get_connections(self, backward: bool = False):
        if self._compressed and backward:
            return [{'forward:y': dim, 'backward:x': dim} for dim in _SHARED_DIMS]
        return []

    def dense_forward(self, *args):
        return self._kernels['forward:y'].dense_func(*args, self._T)


class SparseBatchSoftmaxFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx, sparta_ctx: SparseBatchSoftmaxCtx, x: torch.Tensor):
        ctx.sparta_ctx = sparta_ctx
        y = sparta_ctx.forward(x.detach())
        ctx.save_for_backward(y)
        return y

    @staticmethod
    def backward(ctx, grad: torch.Tensor):
        y, = ctx.saved_tensors
        return None, ctx.sparta_ctx.backward(grad.detach().contiguous(), y.detach())
