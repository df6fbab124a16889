"""Block-sparse matmul kernels: which operand is sparse, which block sizes tile
it, the search space, and the launch closure around spx_matmul.

Interface of sparta/specializer/kernels/matmul.py:21-331.  The mode letters name
A, B, C in that order ('sdd' = sparse A, 'dsd' = sparse B, 'dds' = sparse C).
The two implementation names of the reference are kept as configuration slots:
'sparta' searches block sizes {16,32,64}^3, 'openai' is the fixed 32x64x32
point; both run the same gfx950 MFMA kernels.  The thread-tile look-up table of
the reference has no counterpart: THREAD_SIZE_* values are accepted and ignored.
"""
from typing import Any, Dict, List, Optional

import torch

from sparta_amd import _lib
from sparta_amd.common.tuning import TunableItemCfg
from sparta_amd.specializer.kernels.kernel_base import KernelBase, PortConfig
from sparta_amd.specializer.kernels.operand_sizes import matmul_extent, check_matmul_operands

# mode / transpose -> (sparse port, tile height param, tile width param, index format)
_SPARSE_LAYOUT = {
    ('sdd', False): ('A', 'M', 'K', 'BCSR'),
    ('sdd', True): ('A', 'K', 'M', 'BCSC'),
    ('dsd', True): ('B', 'N', 'K', 'BCSR'),
    ('dsd', False): ('B', 'K', 'N', 'BCSC'),
    ('dds', None): ('C', 'M', 'N', 'BCSR'),
}


class SparseMatMulKernel(KernelBase):

    __algo__: str = ''

    def __init__(self, mode: str, dtype: str = 'float', biased: bool = True,
                 transpose_A: bool = False, transpose_B: bool = True, compressed: bool = True):
        if mode not in ('sdd', 'dsd', 'dds'):
            raise ValueError(f'invalid sparse type: {mode}')
        self._mode = mode
        self._dtype = dtype
        self._biased = biased
        self._transpose_A = transpose_A
        self._transpose_B = transpose_B
        self._compressed = compressed
        key = (mode, {'sdd': transpose_A, 'dsd': transpose_B, 'dds': None}[mode])
        port, tile_h, tile_w, fmt = _SPARSE_LAYOUT[key]
        self._sparse_port = port
        self._sparse_block_H = f'BLOCK_SIZE_{tile_h}_VALUE'
        self._sparse_block_W = f'BLOCK_SIZE_{tile_w}_VALUE'
        self._bcs_mode = fmt
        if fmt == 'BCSR':
            self._tesa_vars = ['row_ptr', 'BCSR_idx', 'nnz']
        else:
            self._tesa_vars = ['col_ptr', 'BCSC_idx', 'nnz']
        if mode == 'dds':
            self._tesa_vars = self._tesa_vars[1:]
        self._epilogue = 0
        super().__init__()

    def set_epilogue(self, activation: Optional[str]):
        """Activation applied by the kernel's own epilogue (an extension: the reference runs a
        separate elementwise kernel after the operator): None or 'relu', sdd / dsd only."""
        if activation not in (None, 'relu'):
            raise ValueError(f'unsupported fused activation: {activation!r}')
        if activation is not None and self._mode == 'dds':
            raise ValueError('the fused activation covers the sdd and dsd kernels only')
        self._epilogue = _lib.EPILOGUE_RELU if activation == 'relu' else 0
        if self.ready:
            self.update_func()

    # ---- ports / parameters -------------------------------------------------------
    def _set_ports(self):
        self.ports['A'] = PortConfig(name='A', is_input=True)
        self.ports['B'] = PortConfig(name='B', is_input=True)
        if self._biased:
            self.ports['bias'] = PortConfig(name='bias', is_input=True)
        self.ports['C'] = PortConfig(name='C', is_input=False)
        self.ports[self._sparse_port].set_sparse(self._bcs_mode == 'BCSR', self._bcs_mode == 'BCSC')

    def _add_parameters(self):
        for name in ('BATCH_SIZE', 'GLOBAL_M_VALUE', 'GLOBAL_K_VALUE', 'GLOBAL_N_VALUE', 'BCSR', 'BCSC'):
            self._add_parameter(name)
        self._add_parameter('BIASED', value=self._biased)
        self._add_parameter('TRANSPOSE_A', value=self._transpose_A)
        self._add_parameter('TRANSPOSE_B', value=self._transpose_B)
        self._add_parameter('COMPRESSED', value=self._compressed)
        # gfx950 tile configuration (0 = chosen from the shape); not part of the
        # default search space so that reference configs and trial counts carry over.
        self._add_parameter('TILE_CFG', value=0)

    def _tile_op(self):
        return _lib.OP_DDS if self._mode == 'dds' else _lib.OP_SPMM

    def set_parameters(self, params: Dict[str, Any]):
        super().set_parameters(params)
        port = self.ports[self._sparse_port]
        if self._bcs_mode == 'BCSR':
            self.set_parameter('BCSR', True)
            self.set_parameter('BCSC', False)
        else:
            self.set_parameter('BCSR', port.BCSR)
            self.set_parameter('BCSC', True)
        port.set_block_size(self.get_parameter(self._sparse_block_H),
                            self.get_parameter(self._sparse_block_W))

    def set_shape(self, batch_size: int, M: int, K: int, N: int):
        self.set_parameter('BATCH_SIZE', batch_size)
        self.set_parameter('GLOBAL_M_VALUE', M)
        self.set_parameter('GLOBAL_K_VALUE', K)
        self.set_parameter('GLOBAL_N_VALUE', N)

    def get_shape(self):
        return tuple(self.get_parameter(n) for n in
                     ('BATCH_SIZE', 'GLOBAL_M_VALUE', 'GLOBAL_K_VALUE', 'GLOBAL_N_VALUE'))

    def get_block_shape(self):
        return tuple(self.get_parameter(f'BLOCK_SIZE_{d}_VALUE') for d in 'MKN')

    def sparse_block_shape(self):
        return (self.ports[self._sparse_port],
                (self.get_parameter(self._sparse_block_H), self.get_parameter(self._sparse_block_W)))

    def blocks_per_grid(self):
        batch_size, M, K, N = self.get_shape()
        if self._mode == 'dds':
            return (self.ports['C'].indexes.block_nnz, batch_size, 1)
        BM, BK, BN = self.get_block_shape()
        return (N // BN, M // BM, batch_size)

    def threads_per_block(self):
        return (256, 1, 1)

    # ---- launch closure ---------------------------------------------------------------
    def update_func(self):
        batch_size, M, K, N = self.get_shape()
        BM, BK, BN = self.get_block_shape()
        indexes = self.ports[self._sparse_port].indexes
        mode_code = _lib.MODE_CODE[self._mode]
        tA, tB = int(self._transpose_A), int(self._transpose_B)
        compressed = int(self._compressed)
        biased = self._biased
        tile_cfg = int(self.get_parameter('TILE_CFG') or 0) | self._epilogue
        tile_elems = self.get_parameter(self._sparse_block_H) * self.get_parameter(self._sparse_block_W)
        lib = _lib.load()

        if self._bcs_mode == 'BCSR':
            ptr, idx, idx_kind = indexes.row_ptr, indexes._bcsr_buf, _lib.IDX_BCSR_I32
        else:
            ptr, idx = indexes.col_ptr, indexes._bcsc_buf
            idx_kind = _lib.IDX_BCSC_I64 if idx.dtype == torch.int64 else _lib.IDX_BCSC_I32
        dds = self._mode == 'dds'
        sched = None if dds else indexes.launch_order('row' if self._bcs_mode == 'BCSR' else 'col')
        sched_p = _lib.dev_ptr(sched)
        # Only a compressed operand / a sparse output need the live block count on the
        # host; a port in at-capacity mode leaves it on the device.
        at_capacity = self.ports[self._sparse_port].at_capacity
        nnz_dev_p = None
        if at_capacity:
            nnz = indexes.capacity
            nnz_dev_p = _lib.dev_ptr(indexes.nnz_dev)
        else:
            nnz = indexes.block_nnz if (compressed or dds) else 0
        sparse_stride = nnz * tile_elems
        if dds and compressed:
            C_shape = (batch_size, nnz * BM * BN)
        else:
            C_shape = (batch_size, M, N)
        # A dense sparse-output result keeps zeros in dead tiles; every other result is
        # fully overwritten by the kernel.
        alloc = torch.zeros if (dds and not compressed) else torch.empty
        ptr_p, idx_p = _lib.dev_ptr(ptr), _lib.dev_ptr(idx)
        # what this closure's kernel walks behind each pointer: a compressed operand laid out
        # by another index (other block shape, other mask) is refused before the launch
        extent = matmul_extent(self._mode, bool(compressed), batch_size, M, K, N, sparse_stride)
        tile = [tile_cfg]   # tile variant (low 16 bits) | epilogue flags; see the retry below

        def matmul_func(A: torch.Tensor, B: torch.Tensor, bias: torch.Tensor = None,
                        _keepalive=(indexes, ptr, idx, sched)):
            assert A.dtype == B.dtype, f'operand dtypes differ: {A.dtype} vs {B.dtype}'
            check_matmul_operands(extent, A, B, bias, biased)
            C = alloc(C_shape, dtype=A.dtype, device=A.device)
            if bias is not None:
                bias = bias.to(A.dtype).contiguous()
            A, B = A.contiguous(), B.contiguous()
            cfg = tile[0]
            while True:
                rc = lib.spx_matmul(
                    mode_code, _lib.dtype_code(A.dtype), tA, tB, compressed,
                    _lib.dev_ptr(A), _lib.dev_ptr(B), _lib.dev_ptr(bias), _lib.dev_ptr(C),
                    ptr_p, idx_p, idx_kind, sched_p, nnz, nnz_dev_p, sparse_stride,
                    batch_size, M, K, N, BM, BK, BN, cfg, _lib.current_stream(A.device))
                if rc == _lib.E_CONFIG and cfg & 0xffff and not self._tile_strict:
                    # the configured tile variant does not take these shapes (nothing was
                    # launched): the library's own choice from here on
                    cfg = tile[0] = cfg & ~0xffff
                    continue
                break
            _lib.check(rc, 'spx_matmul')
            return C

        if biased:
            self._func = lambda A, B, bias: matmul_func(A, B, bias)
        else:
            self._func = lambda A, B: matmul_func(A, B)

    # ---- self test ------------------------------------------------------------------------
    def _convert_data(self, inputs: List[torch.Tensor], outputs: List[torch.Tensor]):
        masked = {'sdd': 0, 'dsd': 1}.get(self._mode)
        if masked is not None:
            inputs[masked] = inputs[masked] * self.ports[self._sparse_port].mask
        for i, x in enumerate(inputs):
            inputs[i] = x.detach()
        outputs[0] = outputs[0].detach()
        if self._compressed:
            indexes = self.ports[self._sparse_port].indexes
            if self._sparse_port == 'C':
                outputs[0] = indexes.convert(outputs[0])
            else:
                inputs[masked] = indexes.convert(inputs[masked],
                                                 at_capacity=self.ports[self._sparse_port].at_capacity)

    def reference(self, *args):
        """Masked-dense result; the sparse-output mode multiplies by the block
        mask the kernel actually computes (a live block is written in full)."""
        A, B = args[0], args[1]
        if self._mode == 'sdd':
            A = A * self.ports['A'].mask
        elif self._mode == 'dsd':
            B = B * self.ports['B'].mask
        lhs = A.transpose(-1, -2) if self._transpose_A else A
        rhs = B.transpose(-1, -2) if self._transpose_B else B
        C = torch.matmul(lhs, rhs)
        if self._biased:
            C = C + args[2].unsqueeze(1)
        if self._epilogue:
            C = torch.relu(C)
        if self._mode == 'dds':
            port = self.ports['C']
            C = C * (port.indexes.get_mask() if self.ready else port.mask)
        return C


class SparTASparseMatMulKernel(SparseMatMulKernel):

    __algo__ = 'sparta'

    def _add_parameters(self):
        super()._add_parameters()
        for dim in 'MKN':
            self._add_parameter(f'BLOCK_SIZE_{dim}_VALUE', is_tunable=True,
                                search_space=TunableItemCfg('choice', [16, 32, 64]))
            self._add_parameter(f'THREAD_SIZE_{dim}_VALUE')

    def _check_parameters(self, params: Dict[str, Any]):
        for dim in 'MKN':
            value = params.get(f'BLOCK_SIZE_{dim}_VALUE')
            assert value in (16, 32, 64), f'BLOCK_SIZE_{dim}_VALUE={value} not in (16, 32, 64)'


class OpenAISparseMatMulKernel(SparseMatMulKernel):

    __algo__ = 'openai'

    _FIXED = {'M': 32, 'K': 64, 'N': 32}

    def _add_parameters(self):
        super()._add_parameters()
        for dim, size in self._FIXED.items():
            self._add_parameter(f'BLOCK_SIZE_{dim}_VALUE', value=size, is_tunable=True,
                                search_space=TunableItemCfg('choice', [size]))

    def _check_parameters(self, params: Dict[str, Any]):
        for dim, size in self._FIXED.items():
            name = f'BLOCK_SIZE_{dim}_VALUE'
            assert params.get(name, size) == size, f'{name} must be {size} for the openai implementation'
