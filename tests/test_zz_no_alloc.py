"""spx_bcs_index_static (the index build whose scratch is a device array inside the
library, for callers that cannot allocate) against spx_bcs_index through the C ABI:
bit-identical outputs on two calls in a row, the second on a smaller mask, and the
size limit is rejected before anything is launched."""
import numpy as np
import pytest
import torch

from oracle import bcs, ops
from sparta_amd import _lib

pytestmark = pytest.mark.gpu


def build(lib, entry, mask, BH, BW, gpu, both):
    H, W = mask.shape
    R, Cn = H // BH, W // BW
    cap = R * Cn
    i32 = dict(dtype=torch.int32, device=gpu)
    out = {'row_ptr': torch.full((R + 1,), -1, **i32), 'bcsr': torch.full((cap,), -1, **i32),
           'nnz': torch.full((1,), -1, **i32)}
    col_ptr = bcsc = None
    if both:
        out['col_ptr'] = col_ptr = torch.full((Cn + 1,), -1, **i32)
        out['bcsc'] = bcsc = torch.full((cap,), -1, dtype=torch.int64, device=gpu)
    args = [_lib.dev_ptr(mask), H, W, BH, BW, _lib.dev_ptr(out['row_ptr']), _lib.dev_ptr(out['bcsr']),
            _lib.dev_ptr(col_ptr), _lib.dev_ptr(bcsc), 1 if both else 0, _lib.dev_ptr(out['nnz']), cap]
    if entry == 'static':
        rc = lib.spx_bcs_index_static(*args, _lib.current_stream(gpu))
    else:
        nbytes = lib.spx_bcs_index_workspace_bytes(H, W, BH, BW)
        ws = torch.empty((nbytes,), dtype=torch.uint8, device=gpu)
        rc = lib.spx_bcs_index(*args, _lib.dev_ptr(ws), nbytes, _lib.current_stream(gpu))
    _lib.check(rc, f'spx_bcs_index ({entry})')
    torch.cuda.synchronize()
    nnz = int(out['nnz'].item())
    out['bcsr'] = out['bcsr'][:nnz]
    if both:
        out['bcsc'] = out['bcsc'][:nnz]
    return out


@pytest.mark.parametrize('both', [False, True])
def test_static_index_matches_workspace_index_twice(both, gpu):
    lib = _lib.load()
    # first call: a 2048 x 4096 mask in 16 x 32 blocks; second call: a smaller mask in other blocks,
    # which leaves most of the first call's scratch contents in place
    cases = [((2048, 4096), (16, 32), (8, 8), 0.9, 1), ((384, 320), (32, 64), (1, 1), 0.999, 2)]
    for shape, (BH, BW), gran, sparsity, seed in cases:
        mask_np = ops.block_mask(shape, gran, sparsity, seed=seed)
        mask = torch.from_numpy(mask_np).to(gpu)
        got = build(lib, 'static', mask, BH, BW, gpu, both)
        want = build(lib, 'workspace', mask, BH, BW, gpu, both)
        assert got.keys() == want.keys()
        for name in want:
            assert torch.equal(got[name], want[name]), f'{name} differs for mask {shape} in {BH}x{BW} blocks'
        row_ptr, idx, nnz = bcs.build_bcsr(mask_np, BH, BW)
        assert int(got['nnz'].item()) == nnz
        assert np.array_equal(got['row_ptr'].cpu().numpy(), row_ptr)
        assert np.array_equal(got['bcsr'].cpu().numpy(), idx)


def test_static_index_rejects_masks_beyond_its_scratch(gpu):
    lib = _lib.load()
    limit = lib.spx_bcs_index_static_max_bytes()
    H = W = 4096
    assert lib.spx_bcs_index_workspace_bytes(H, W, 4, 4) > limit
    mask = torch.zeros((H, W), dtype=torch.uint8, device=gpu)
    R = H // 4
    i32 = dict(dtype=torch.int32, device=gpu)
    row_ptr, bcsr, nnz = torch.zeros((R + 1,), **i32), torch.zeros((16,), **i32), torch.zeros((1,), **i32)
    rc = lib.spx_bcs_index_static(_lib.dev_ptr(mask), H, W, 4, 4, _lib.dev_ptr(row_ptr), _lib.dev_ptr(bcsr),
                                  None, None, 0, _lib.dev_ptr(nnz), 16, _lib.current_stream(gpu))
    assert rc == _lib.E_WORKSPACE
    assert 'static buffer' in _lib.last_error()
