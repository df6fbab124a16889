"""Masked block-sparse softmax kernels (forward / backward).

Interface of sparta/specializer/kernels/softmax.py:17-210.  x, y (and the
gradients) share one BCSR index; `T` handed to the kernels is 1/temperature.
"""
from typing import Any, Dict, List, Tuple

import numpy as np
import torch

from sparta_amd import _lib
from sparta_amd.common.tuning import TunableItemCfg
from sparta_amd.specializer.kernels.kernel_base import KernelBase, PortConfig
from sparta_amd.specializer.kernels.operand_sizes import require_numel
from sparta_amd.testing import sparse_softmax_forward_reference, sparse_softmax_backward_reference


class SparseSoftmaxKernel(KernelBase):

    __algo__: str = ''
    __direction__: str = ''

    def __init__(self, compressed: bool = False, dtype: str = 'float'):
        self._compressed = compressed
        self._dtype = dtype
        super().__init__()

    def _add_parameters(self):
        for name in ('BATCH_SIZE', 'GLOBAL_H_VALUE', 'GLOBAL_W_VALUE'):
            self._add_parameter(name)
        self._add_parameter('COMPRESSED', value=self._compressed)
        # gfx950 kernel variant (0 = chosen by the library); outside the default search space
        self._add_parameter('TILE_CFG', value=0)

    def _tile_op(self):
        return _lib.OP_SOFTMAX

    def set_parameters(self, params: Dict[str, Any]):
        super().set_parameters(params)
        self.ports['y'].set_block_size(*self.get_block_shape())

    def set_shape(self, batch_size: int, H: int, W: int):
        self.set_parameter('BATCH_SIZE', batch_size)
        self.set_parameter('GLOBAL_H_VALUE', H)
        self.set_parameter('GLOBAL_W_VALUE', W)

    def get_shape(self):
        return tuple(self.get_parameter(n) for n in ('BATCH_SIZE', 'GLOBAL_H_VALUE', 'GLOBAL_W_VALUE'))

    def get_block_shape(self):
        return self.get_parameter('BLOCK_SIZE_H_VALUE'), self.get_parameter('BLOCK_SIZE_W_VALUE')

    def sparse_block_shape(self):
        return self.ports['y'], self.get_block_shape()

    def _launch_state(self):
        """Everything a launch closure needs, resolved once per update_func()."""
        batch_size, H, W = self.get_shape()
        BH, BW = self.get_block_shape()
        indexes = self.ports['y'].indexes
        mask = indexes.raw_mask
        tile_cfg = int(self.get_parameter('TILE_CFG') or 0)
        if self._compressed:
            shape = (batch_size, indexes.block_nnz * BH * BW)
        else:
            shape = (batch_size, H, W)
        # A mask that is uniform inside its blocks needs no per-entry test: the kernel
        # takes NULL for "every entry of a live block takes part" (one synchronising
        # comparison per index build).
        if not self.ports['y'].at_capacity and indexes.is_block_uniform():
            mask = None
        elif self._compressed:
            mask = indexes.convert(mask)
        stride = int(np.prod(shape[1:]))
        if tile_cfg == 0 and not self.ports['y'].at_capacity and BW % 8 == 0:
            # short rows (known from the live block count): sixteen lanes per row
            if indexes.block_nnz * BW <= 410 * max(indexes.row_num, 1):
                tile_cfg = 3
        return batch_size, H, W, BH, BW, indexes, mask, shape, stride, tile_cfg

    def _mask_and_compress(self, tensors: List[torch.Tensor], positions: List[int]):
        mask = self.ports['y'].mask
        for i in positions:
            tensors[i] = (tensors[i].reshape(self.get_shape()) * mask).detach()
            if self._compressed:
                tensors[i] = self.ports['y'].indexes.convert(tensors[i])


class SparseSoftmaxForwardKernel(SparseSoftmaxKernel):

    __direction__ = 'forward'

    def _set_ports(self):
        self.ports['x'] = PortConfig(name='x', is_input=True, is_sparse=True, BCSR=True)
        self.ports['y'] = PortConfig(name='y', is_input=False, is_sparse=True, BCSR=True)
        self.ports['x'].connect(self, 'y')

    def update_func(self):
        batch_size, H, W, BH, BW, indexes, mask, shape, stride, tile_cfg = self._launch_state()
        compressed = int(self._compressed)
        alloc = torch.empty if self._compressed else torch.zeros
        row_ptr, idx = indexes.row_ptr, indexes._bcsr_buf
        lib = _lib.load()

        numel = batch_size * stride
        tile = [tile_cfg]
        if mask is not None:
            require_numel('spx_softmax_forward', 'mask', mask, stride)

        def softmax_forward_func(x: torch.Tensor, T: np.float32):
            require_numel('spx_softmax_forward', 'x', x, numel)
            y = alloc(shape, dtype=x.dtype, device=x.device)
            if y.numel() == 0:  # no live block: nothing to compute
                return y
            x = x.contiguous()
            while True:
                rc = lib.spx_softmax_forward(
                    _lib.dtype_code(x.dtype), compressed, _lib.dev_ptr(x), _lib.dev_ptr(y),
                    _lib.dev_ptr(row_ptr), _lib.dev_ptr(idx), _lib.dev_ptr(mask), float(T),
                    batch_size, H, W, BH, BW, stride, tile[0], _lib.current_stream(x.device))
                if rc == _lib.E_CONFIG and tile[0] and not self._tile_strict:
                    tile[0] = 0   # the configured variant does not take this dtype / block width
                    continue
                break
            _lib.check(rc, 'spx_softmax_forward')
            return y

        self._func = softmax_forward_func

    def _convert_data(self, inputs, outputs):
        self._mask_and_compress(inputs, [0])
        self._mask_and_compress(outputs, [0])

    def reference(self, *args):
        x, T = args
        return sparse_softmax_forward_reference(x, self.ports['y'].mask, 1 / T)


class SparseSoftmaxBackwardKernel(SparseSoftmaxKernel):

    __direction__ = 'backward'

    def _set_ports(self):
        self.ports['grad_y'] = PortConfig(name='grad_y', is_input=True, is_sparse=True, BCSR=True)
        self.ports['y'] = PortConfig(name='y', is_input=True, is_sparse=True, BCSR=True)
        self.ports['grad_x'] = PortConfig(name='grad_x', is_input=False, is_sparse=True, BCSR=True)
        self.ports['grad_y'].connect(self, 'y')
        self.ports['grad_y'].connect(self, 'grad_x')

    def update_func(self):
        batch_size, H, W, BH, BW, indexes, mask, shape, stride, tile_cfg = self._launch_state()
        compressed = int(self._compressed)
        alloc = torch.empty if self._compressed else torch.zeros
        row_ptr, idx = indexes.row_ptr, indexes._bcsr_buf
        lib = _lib.load()

        numel = batch_size * stride
        tile = [tile_cfg]
        if mask is not None:
            require_numel('spx_softmax_backward', 'mask', mask, stride)

        def softmax_backward_func(grad_y: torch.Tensor, y: torch.Tensor, T: np.float32):
            require_numel('spx_softmax_backward', 'grad_y', grad_y, numel)
            require_numel('spx_softmax_backward', 'y', y, numel)
            assert grad_y.dtype == y.dtype, f'operand dtypes differ: {grad_y.dtype} vs {y.dtype}'
            grad_x = alloc(shape, dtype=grad_y.dtype, device=grad_y.device)
            if grad_x.numel() == 0:
                return grad_x
            grad_y, y = grad_y.contiguous(), y.contiguous()
            while True:
                rc = lib.spx_softmax_backward(
                    _lib.dtype_code(grad_y.dtype), compressed, _lib.dev_ptr(grad_y), _lib.dev_ptr(y), _lib.dev_ptr(grad_x),
                    _lib.dev_ptr(row_ptr), _lib.dev_ptr(idx), _lib.dev_ptr(mask), float(T),
                    batch_size, H, W, BH, BW, stride, tile[0], _lib.current_stream(grad_y.device))
                if rc == _lib.E_CONFIG and tile[0] and not self._tile_strict:
                    tile[0] = 0
                    continue
                break
            _lib.check(rc, 'spx_softmax_backward')
            return grad_x

        self._func = softmax_backward_func

    def _convert_data(self, inputs, outputs):
        self._mask_and_compress(inputs, [0, 1])
        self._mask_and_compress(outputs, [0])

    def reference(self, *args):
        grad_y, y, T = args
        return sparse_softmax_backward_reference(grad_y, y, self.ports['y'].mask, 1 / T)


class SparTASoftmaxKernel(SparseSoftmaxKernel):

    __algo__ = 'sparta'

    def _add_parameters(self):
        super()._add_parameters()
        for name, values in (('BLOCK_SIZE_H_VALUE', [8, 16, 32, 64, 128]),
                             ('BLOCK_SIZE_W_VALUE', [16, 32, 64, 128]),
                             ('ROW_TILE_VALUE', [1, 2, 4, 8, 16])):
            self._add_parameter(name, is_tunable=True, search_space=TunableItemCfg('choice', values))

    def blocks_per_grid(self):
        batch_size, H, W = self.get_shape()
        return ((H + 3) // 4, batch_size, 1)

    def threads_per_block(self) -> Tuple[int, ...]:
        return (256, 1, 1)

    def _check_parameters(self, params: Dict[str, Any]):
        # The reference requires BLOCK_SIZE_H_VALUE > ROW_TILE_VALUE
        # (softmax.py:191-195); keep the rule so the same configs are rejected.
        assert params['BLOCK_SIZE_H_VALUE'] > params['ROW_TILE_VALUE'], \
            'BLOCK_SIZE_H_VALUE must exceed ROW_TILE_VALUE'


class SparTASparseSoftmaxForwardKernel(SparseSoftmaxForwardKernel, SparTASoftmaxKernel):
    pass


class SparTASparseSoftmaxBackwardKernel(SparseSoftmaxBackwardKernel, SparTASoftmaxKernel):
    pass
