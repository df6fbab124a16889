"""ctypes binding of libsparta_hip.so (the C ABI declared in include/sparta_hip.h).

The library is the only compute path of this package: if it is missing the
import of any operator fails loudly instead of falling back to PyTorch.
"""
import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'lib', 'libsparta_hip.so')

# enums of include/sparta_hip.h
F32, F16, BF16 = 0, 1, 2
SDD, DSD, DDS = 0, 1, 2
IDX_BCSR_I32, IDX_BCSC_I32, IDX_BCSC_I64 = 0, 1, 2
EPILOGUE_RELU = 0x10000   # or-ed into spx_matmul's tile_cfg
E_NULL, E_SHAPE, E_DTYPE, E_ALIGN, E_WORKSPACE, E_CONFIG, E_NO_DEVICE = -1, -2, -3, -4, -5, -6, -7
OP_SPMM, OP_DDS, OP_SOFTMAX, OP_ATTENTION, OP_MOE = 0, 1, 2, 3, 4

MODE_CODE = {'sdd': SDD, 'dsd': DSD, 'dds': DDS}
_DTYPE_CODE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}


class TileCfg(ctypes.Structure):
    _fields_ = [
        ('id', ctypes.c_int), ('tile_m', ctypes.c_int), ('tile_n', ctypes.c_int),
        ('waves', ctypes.c_int), ('lds_stages', ctypes.c_int), ('min_block', ctypes.c_int),
        ('dtype_mask', ctypes.c_int), ('name', ctypes.c_char * 32),
    ]


_c = ctypes
_P, _I, _L, _F, _Z = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_float, _c.c_size_t


class BcsIndexJob(ctypes.Structure):
    """spx_bcs_index_job: the arguments of spx_bcs_index_scheduled for one mask."""
    _fields_ = [
        ('mask', _P), ('H', _I), ('W', _I), ('BH', _I), ('BW', _I),
        ('row_ptr', _P), ('bcsr_idx', _P), ('col_ptr', _P), ('bcsc_idx', _P), ('bcsc_i64', _I),
        ('nnz_dev', _P), ('cap', _I), ('row_order', _P), ('col_order', _P),
        ('workspace', _P), ('workspace_bytes', _Z),
    ]


_SIGNATURES = {
    'spx_last_error': (_c.c_char_p, []),
    'spx_version': (_I, []),
    'spx_stream_probe': (_I, [_I, _P, _P, _Z, _P]),
    'spx_bcs_index_workspace_bytes': (_Z, [_I, _I, _I, _I]),
    'spx_bcs_index': (_I, [_P, _I, _I, _I, _I, _P, _P, _P, _P, _I, _P, _I, _P, _Z, _P]),
    'spx_bcs_index_scheduled': (_I, [_P, _I, _I, _I, _I, _P, _P, _P, _P, _I, _P, _I, _P, _P, _P, _Z, _P]),
    'spx_bcs_index_batch': (_I, [_c.POINTER(BcsIndexJob), _I, _P]),
    'spx_bcs_index_static_max_bytes': (_Z, []),
    'spx_bcs_index_static': (_I, [_P, _I, _I, _I, _I, _P, _P, _P, _P, _I, _P, _I, _P]),
    'spx_bcs_gather': (_I, [_P, _P, _P, _I, _I, _P, _I, _I, _I, _I, _I, _I, _L, _P]),
    'spx_bcs_scatter': (_I, [_P, _P, _P, _I, _I, _P, _I, _I, _I, _I, _I, _I, _L, _P]),
    'spx_bcs_sum': (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _L, _P]),
    'spx_bcs_schedule': (_I, [_P, _I, _P, _P]),
    'spx_matmul': (_I, [_I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _I, _P, _I, _P, _L,
                        _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    'spx_softmax_forward': (_I, [_I, _I, _P, _P, _P, _P, _P, _F, _I, _I, _I, _I, _I, _L, _I, _P]),
    'spx_softmax_backward': (_I, [_I, _I, _P, _P, _P, _P, _P, _P, _F, _I, _I, _I, _I, _I, _L, _I, _P]),
    'spx_attention_forward': (_I, [_I, _P, _P, _P, _P, _P, _P, _P, _F, _I, _I, _I, _I, _I, _I, _I, _P]),
    'spx_attention_forward_train': (_I, [_I, _P, _P, _P, _P, _P, _L, _P, _P, _P, _F, _I, _I, _I, _I, _I, _I, _P]),
    'spx_attention_backward_scores': (_I, [_I, _P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _P, _F, _I, _I, _I, _I, _I, _I, _P]),
    'spx_attention_backward_kv': (_I, [_I, _P, _P, _P, _P, _P, _P, _P, _L, _P, _P, _I, _F, _I, _I, _I, _I, _I, _I, _P]),
    'spx_attention_forward_lse': (_I, [_I, _P, _P, _P, _P, _P, _P, _P, _P, _F, _I, _I, _I, _I, _I, _I, _P]),
    'spx_attention_backward_q': (_I, [_I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _F, _I, _I, _I, _I, _I, _I, _P]),
    'spx_attention_backward_kv_recompute': (_I, [_I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _F, _I, _I, _I, _I, _I, _I, _P]),
    'spx_attention_seqlen_forward': (_I, [_I, _P, _P, _P, _P, _P, _F, _I, _I, _I, _I, _I, _P]),
    'spx_moe_index_workspace_bytes': (_Z, [_I, _I]),
    'spx_moe_index': (_I, [_P, _I, _I, _P, _P, _P, _P, _Z, _P]),
    'spx_moe_forward': (_I, [_I, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    'spx_num_tile_cfgs': (_I, [_I]),
    'spx_tile_cfg_info': (_I, [_I, _I, _c.POINTER(TileCfg)]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f'{LIB_PATH} is missing: the HIP extension has not been built. '
                'Run `python -m sparta_amd.build` (needs hipcc); there is no fallback path.'
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def last_error() -> str:
    return load().spx_last_error().decode()


def check(rc: int, what: str):
    """Map a return code to the exception convention of the reference:
    invalid shape / tile combinations are AssertionError (the tuner skips such
    trials), everything else is a hard error."""
    if rc == 0:
        return
    msg = f'{what}: {last_error()} (code {rc})'
    if rc in (E_SHAPE, E_CONFIG):
        raise AssertionError(msg)
    if rc in (E_NULL, E_DTYPE, E_ALIGN, E_WORKSPACE):
        raise ValueError(msg)
    raise RuntimeError(msg)


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f'unsupported dtype {dtype}: expected float32, float16 or bfloat16')


def dev_ptr(t: Optional[torch.Tensor]):
    """Device address of a contiguous GPU tensor (None -> NULL)."""
    if t is None:
        return None
    if not t.is_cuda:
        raise RuntimeError('sparta_amd kernels run on the GPU only: got a CPU tensor')
    if not t.is_contiguous():
        raise ValueError('sparta_amd kernels need contiguous tensors')
    return _c.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def current_stream(device=None):
    """The current stream of `device` as a C pointer.  A torch.device with an index takes the
    short way (no Stream object is built: this runs once per kernel launch)."""
    if _raw_stream is not None and isinstance(device, torch.device) and device.index is not None:
        return _c.c_void_p(_raw_stream(device.index))
    return _c.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def tile_configs(op: int):
    lib = load()
    out = []
    for i in range(lib.spx_num_tile_cfgs(op)):
        cfg = TileCfg()
        check(lib.spx_tile_cfg_info(op, i, ctypes.byref(cfg)), 'spx_tile_cfg_info')
        out.append({
            'id': cfg.id, 'tile_m': cfg.tile_m, 'tile_n': cfg.tile_n, 'waves': cfg.waves,
            'lds_stages': cfg.lds_stages, 'min_block': cfg.min_block,
            'dtype_mask': cfg.dtype_mask, 'name': cfg.name.decode(),
        })
    return out
