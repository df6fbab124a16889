"""GPU parity of the masked block-sparse softmax (forward / backward) against the
numpy oracle.  Base case from the reference's test/unit/test_sparse_softmax.py:53-59
(H=128, W=256, 8x8-granular 90% mask, temperature sqrt(W), blocks 32x32)."""
import numpy as np
import pytest
import torch

from oracle import bcs, ops
from sparta_amd.specializer.kernels import SparTASparseSoftmaxForwardKernel, SparTASparseSoftmaxBackwardKernel
from helpers import randn, assert_close

pytestmark = pytest.mark.gpu


def build(cls, mask, batch, H, W, BH, BW, compressed, tile_cfg=0):
    kernel = cls(compressed=compressed)
    kernel.ports['y'].set_mask(mask)
    kernel.set_shape(batch, H, W)
    kernel.compile({'BLOCK_SIZE_H_VALUE': BH, 'BLOCK_SIZE_W_VALUE': BW, 'ROW_TILE_VALUE': 4, 'TILE_CFG': tile_cfg})
    return kernel


@pytest.mark.parametrize('compressed', [False, True])
@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize('BH,BW', [(32, 32), (8, 16), (64, 128), (16, 64), (16, 4)])
@pytest.mark.parametrize('tile_cfg,gran', [(0, (8, 8)), (1, (8, 8)), (2, (8, 8)), (3, (8, 8)), (0, None), (2, (1, 1)), (3, (1, 1))])
def test_softmax_forward_backward(compressed, dtype, BH, BW, tile_cfg, gran, gpu, batch=4, H=128, W=256):
    """gran None: the mask is uniform inside the kernel's blocks (no per-entry mask is
    passed); (1, 1): element-granular.  tile_cfg 2 needs 16 bytes of entries per block row."""
    if tile_cfg >= 2 and BW * (4 if dtype == torch.float32 else 2) < 16:
        pytest.skip('block row shorter than one 16-byte access')
    T = float(np.sqrt(W))
    x_np, x_t = randn((batch, H, W), 7, dtype, scale=4.0)
    g_np, g_t = randn((batch, H, W), 8, dtype)
    mask_np = ops.block_mask((H, W), gran or (BH, BW), 0.9 if gran != (1, 1) else 0.6, seed=2022)
    mask_np[32:48, :] = 0  # a band of fully masked rows
    mask = torch.from_numpy(mask_np).to(gpu)
    fwd = build(SparTASparseSoftmaxForwardKernel, mask, batch, H, W, BH, BW, compressed, tile_cfg)
    bwd = build(SparTASparseSoftmaxBackwardKernel, mask, batch, H, W, BH, BW, compressed, tile_cfg)
    idx = fwd.ports['y'].indexes
    want_y = ops.softmax_forward_reference(x_np, mask_np, T)

    x = x_t.to(gpu) * mask.to(dtype)
    x_in = idx.convert(x) if compressed else x
    y = fwd(x_in, np.float32(1 / T))
    y_dense = idx.inverse(y) if compressed else y
    assert_close(y_dense, want_y, dtype, 'softmax forward')
    assert float(y_dense[:, 32:48].abs().max()) == 0.0

    # backward on the dtype-rounded forward result so both sides see the same y
    y_round = y_dense.to(torch.float64).cpu().numpy()
    want_gx = ops.softmax_backward_reference(g_np, y_round, mask_np, T)
    g = g_t.to(gpu) * mask.to(dtype)
    g_in = idx.convert(g) if compressed else g
    gx = bwd(g_in, y, np.float32(1 / T))
    gx_dense = idx.inverse(gx) if compressed else gx
    assert_close(gx_dense, want_gx, dtype, 'softmax backward')


def test_softmax_long_rows(gpu):
    """Rows with more live entries than the register cache holds (> 1024)."""
    H, W = 64, 4096
    x_np, x_t = randn((2, H, W), 3, torch.float32, scale=3.0)
    mask_np = ops.block_mask((H, W), (1, 1), 0.3, seed=4)
    mask = torch.from_numpy(mask_np).to(gpu)
    for tile_cfg in (1, 2, 3):
        fwd = build(SparTASparseSoftmaxForwardKernel, mask, 2, H, W, 32, 64, False, tile_cfg)
        y = fwd(x_t.to(gpu), np.float32(0.5))
        assert_close(y, ops.softmax_forward_reference(x_np, mask_np, 2.0), torch.float32, f'long rows cfg {tile_cfg}')
        np.testing.assert_allclose(y.sum(-1).cpu().numpy(), 1.0, rtol=1e-5)


def test_softmax_all_ones_mask_matches_torch(gpu):
    x = torch.randn((3, 64, 128), generator=torch.Generator().manual_seed(0))
    mask = torch.ones((64, 128), dtype=torch.uint8, device=gpu)
    fwd = build(SparTASparseSoftmaxForwardKernel, mask, 3, 64, 128, 16, 32, False)
    y = fwd(x.to(gpu), np.float32(1.0))
    torch.testing.assert_close(y.cpu(), torch.softmax(x, -1), rtol=1e-5, atol=1e-6)
