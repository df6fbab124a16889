"""GPU parity of the block-sparse matmul kernels against the numpy oracle.
Cases follow the reference's test/unit/test_sparse_matmul.py:98-174 (batch 4,
M=128, K=256, N=192, 8x8-granular mask at 90%) over every mode, transpose,
bias and storage variant, both implementation slots and three dtypes."""
import itertools

import numpy as np
import pytest
import torch

from oracle import bcs, ops
from sparta_amd.specializer.kernels import SparTASparseMatMulKernel, OpenAISparseMatMulKernel
from helpers import randn, assert_close

pytestmark = pytest.mark.gpu


def run_case(gpu, mode, tA, tB, biased, compressed, dtype, blocks, impl='sparta',
             batch=4, M=128, K=256, N=192, gran=(8, 8), sparsity=0.9, seed=2022, tile_cfg=0, activation=None):
    BM, BK, BN = blocks
    A_shape = (K, M) if tA else (M, K)
    B_shape = (N, K) if tB else (K, N)
    a_np, a_t = randn((batch,) + A_shape, seed, dtype)
    b_np, b_t = randn((batch,) + B_shape, seed + 1, dtype)
    bias_np, bias_t = randn((batch, N), seed + 2, dtype)
    mask_shape = {'sdd': A_shape, 'dsd': B_shape, 'dds': (M, N)}[mode]
    mask_np = ops.block_mask(mask_shape, gran, sparsity, seed=seed + 3)
    mask = torch.from_numpy(mask_np).to(gpu)

    cls = SparTASparseMatMulKernel if impl == 'sparta' else OpenAISparseMatMulKernel
    kernel = cls(mode=mode, biased=biased, transpose_A=tA, transpose_B=tB, compressed=compressed)
    port = {'sdd': 'A', 'dsd': 'B', 'dds': 'C'}[mode]
    kernel.ports[port].set_mask(mask)
    kernel.set_shape(batch, M, K, N)
    kernel.compile({'BLOCK_SIZE_M_VALUE': BM, 'BLOCK_SIZE_K_VALUE': BK, 'BLOCK_SIZE_N_VALUE': BN,
                    'TILE_CFG': tile_cfg})
    if activation is not None:
        kernel.set_epilogue(activation)
    indexes = kernel.ports[port].indexes
    tile = {'sdd': (BK, BM) if tA else (BM, BK), 'dsd': (BN, BK) if tB else (BK, BN), 'dds': (BM, BN)}[mode]
    assert (indexes.block_H, indexes.block_W) == tile

    want = ops.matmul_reference(a_np, b_np, bias_np if biased else None, mode=mode, transpose_A=tA,
                                transpose_B=tB, mask=mask_np, block=tile, dtype=np.float64)
    if activation == 'relu':
        want = np.maximum(want, 0.0)
    A = a_t.to(gpu)
    B = b_t.to(gpu)
    # masked operands go in masked (the kernel reads every element of a live block)
    if mode == 'sdd':
        A = A * mask.to(dtype)
        if compressed:
            A = indexes.convert(A)
    elif mode == 'dsd':
        B = B * mask.to(dtype)
        if compressed:
            B = indexes.convert(B)
    args = [A, B] + ([bias_t.to(gpu)] if biased else [])
    C = kernel(*args)
    if mode == 'dds' and compressed:
        fmt_idx = indexes.BCSR_idx.cpu().numpy()
        want = bcs.convert(want, fmt_idx, 'bcsr', BM, BN)
    assert C.dtype == dtype and tuple(C.shape) == want.shape
    assert_close(C, want, dtype, f'{mode} tA={tA} tB={tB} bias={biased} comp={compressed} {dtype}')


@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
@pytest.mark.parametrize('tA', [False, True])
@pytest.mark.parametrize('tB', [False, True])
@pytest.mark.parametrize('compressed', [False, True])
@pytest.mark.parametrize('biased', [False, True])
def test_matmul_fp32_all_variants(mode, tA, tB, compressed, biased, gpu):
    run_case(gpu, mode, tA, tB, biased, compressed, torch.float32, (32, 32, 32))


@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
@pytest.mark.parametrize('tA', [False, True])
@pytest.mark.parametrize('tB', [False, True])
@pytest.mark.parametrize('compressed', [False, True])
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_matmul_half_all_variants(mode, tA, tB, compressed, dtype, gpu):
    run_case(gpu, mode, tA, tB, True, compressed, dtype, (32, 32, 32))


@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
@pytest.mark.parametrize('tA,tB', [(False, True), (True, False)])
@pytest.mark.parametrize('dtype', [torch.float32, torch.float16])
def test_matmul_openai_slot(mode, tA, tB, dtype, gpu):
    run_case(gpu, mode, tA, tB, True, True, dtype, (32, 64, 32), impl='openai')


BLOCKS = [b for b in itertools.product([16, 32, 64], repeat=3)]


@pytest.mark.parametrize('blocks', BLOCKS)
@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
def test_matmul_block_shapes(blocks, mode, gpu):
    # alternate dtype / transposes over the 27 block shapes to keep the suite short
    k = BLOCKS.index(blocks)
    dtype = [torch.float32, torch.float16, torch.bfloat16][k % 3]
    run_case(gpu, mode, bool(k & 1), bool(k & 2), bool(k & 4), bool(k & 8), dtype, blocks,
             batch=2, M=192, K=128, N=256, gran=(16, 16), sparsity=0.8, seed=k)


@pytest.mark.parametrize('tile_cfg', [1, 2, 3, 4, 5, 6, 7, 8, 10])
@pytest.mark.parametrize('mode', ['sdd', 'dsd'])
@pytest.mark.parametrize('compressed', [False, True])
@pytest.mark.parametrize('dtype,blocks', [(torch.float16, (32, 32, 32)), (torch.bfloat16, (64, 64, 32)),
                                          (torch.float32, (16, 16, 64)), (torch.float16, (32, 64, 16)),
                                          (torch.float32, (32, 32, 32))])
def test_matmul_tile_configs(tile_cfg, mode, compressed, dtype, blocks, gpu):
    """Every kernel family behind TILE_CFG gives the same masked-dense result
    (k-contiguous layout, which all of them accept); M is ragged on purpose."""
    if tile_cfg == 8 and (blocks[2] if mode == 'dsd' else blocks[0]) > 32:
        pytest.skip('the K-split kernel covers sparse-side block widths up to 32')
    run_case(gpu, mode, False, True, True, compressed, dtype, blocks, batch=2,
             M=320 if mode == 'dsd' else 192, K=256, N=192 if mode == 'dsd' else 328, gran=(16, 16),
             sparsity=0.7, seed=11, tile_cfg=tile_cfg)


@pytest.mark.parametrize('tile_cfg', [0, 1, 2, 3, 4, 5, 6, 7, 8, 10])
@pytest.mark.parametrize('mode', ['sdd', 'dsd'])
@pytest.mark.parametrize('biased', [False, True])
@pytest.mark.parametrize('dtype,blocks', [(torch.float16, (32, 32, 32)), (torch.bfloat16, (32, 64, 32)),
                                          (torch.float32, (16, 16, 16))])
def test_matmul_fused_relu(tile_cfg, mode, biased, dtype, blocks, gpu):
    """SPX_EPILOGUE_RELU or-ed into the tile config: every kernel family of the sparse-operand
    product clamps its result (after the bias) at zero in its own epilogue."""
    run_case(gpu, mode, False, True, biased, True, dtype, blocks, batch=2,
             M=320 if mode == 'dsd' else 192, K=256, N=192 if mode == 'dsd' else 328, gran=(16, 16),
             sparsity=0.7, seed=29, tile_cfg=tile_cfg, activation='relu')


def test_matmul_fused_relu_thin_operand_and_rejections(gpu):
    run_case(gpu, 'sdd', False, False, True, True, torch.float16, (64, 32, 32), batch=5, M=448, K=320, N=64,
             gran=(32, 32), sparsity=0.8, seed=31, tile_cfg=9, activation='relu')
    kernel = SparTASparseMatMulKernel(mode='dds', biased=False, transpose_A=False, transpose_B=True, compressed=True)
    with pytest.raises(ValueError):
        kernel.set_epilogue('relu')
    with pytest.raises(ValueError):
        SparTASparseMatMulKernel(mode='dsd').set_epilogue('gelu')


@pytest.mark.parametrize('mode', ['sdd', 'dsd'])
@pytest.mark.parametrize('compressed', [False, True])
@pytest.mark.parametrize('dtype,blocks', [(torch.float16, (32, 32, 32)), (torch.bfloat16, (64, 64, 64)),
                                          (torch.float32, (16, 16, 16)), (torch.float16, (32, 64, 32))])
def test_matmul_persistent_kernel_walks_several_tiles(mode, compressed, dtype, blocks, gpu):
    """Tile config 10 with seventeen 256-row tiles of the dense operand, the last one
    partial: three tiles for the workgroups of the first XCD, two for the others; block
    columns of zero, one (odd step count) and several live blocks; both output layouts."""
    dense_rows = 16 * 256 + 104 if mode == 'dsd' else 16 * 256 + 128
    M, N = (dense_rows, 192) if mode == 'dsd' else (192, dense_rows)
    run_case(gpu, mode, False, True, True, compressed, dtype, blocks, batch=2, M=M, K=256, N=N,
             gran=blocks[:2] if mode == 'sdd' else (blocks[2], blocks[1]), sparsity=0.75, seed=17, tile_cfg=10)


@pytest.mark.parametrize('compressed', [False, True])
@pytest.mark.parametrize('dtype,blocks', [(torch.float16, (32, 32, 32)), (torch.bfloat16, (16, 32, 64)),
                                          (torch.float32, (32, 16, 16))])
def test_matmul_persistent_kernel_sparse_operand_stored_the_other_way(compressed, dtype, blocks, gpu):
    """Tile config 10 with the sparse operand stored with its non-reduced dimension contiguous
    (weight [K, N], transpose_B = False; sparse input [K, M], transpose_A = True): its blocks
    are turned on their way into LDS."""
    rows = 3 * 256 + 72
    run_case(gpu, 'dsd', False, False, True, compressed, dtype, blocks, batch=2, M=rows, K=256, N=192,
             gran=(blocks[1], blocks[2]), sparsity=0.7, seed=41, tile_cfg=10)
    run_case(gpu, 'sdd', True, True, True, compressed, dtype, blocks, batch=2, M=192, K=256, N=rows,
             gran=(blocks[1], blocks[0]), sparsity=0.7, seed=43, tile_cfg=10)


@pytest.mark.parametrize('mode', ['sdd', 'dsd'])
@pytest.mark.parametrize('dtype', [torch.float16, torch.float32])
def test_matmul_persistent_kernel_long_operand_in_several_launches(mode, dtype, gpu):
    """Tile config 10 walks a dense operand of more than thirty-two 256-row tiles in several
    launches: thirty-four tiles here, the last one partial, with a bias (which runs along the
    chunked dimension in one of the two modes)."""
    dense_rows = 33 * 256 + 40
    M, N = (dense_rows, 64) if mode == 'dsd' else (64, dense_rows)
    run_case(gpu, mode, False, True, True, True, dtype, (32, 32, 32), batch=2, M=M, K=128, N=N,
             gran=(32, 32), sparsity=0.5, seed=37, tile_cfg=10)


@pytest.mark.parametrize('mode', ['sdd', 'dsd'])
@pytest.mark.parametrize('case', ['long columns', 'many columns'])
def test_matmul_persistent_kernel_index_paths(mode, case, gpu):
    """Tile config 10 off its common path: block columns of more than 64 live blocks (the entries
    past the 64 that sit in a lane vector are read from the index at their step), and more than
    128 block columns (launch order and column pointers are read per tile instead of sitting in
    lane vectors)."""
    if case == 'long columns':
        blocks, sparse_rows, K, sparsity = (16, 32, 16), 64, 32 * 88, 0.12
    else:
        blocks, sparse_rows, K, sparsity = (16, 32, 16), 16 * 150, 128, 0.6
    M, N = (600, sparse_rows) if mode == 'dsd' else (sparse_rows, 600)
    run_case(gpu, mode, False, True, True, True, torch.float16, blocks, batch=1, M=M, K=K, N=N,
             gran=(16, blocks[1]), sparsity=sparsity, seed=23, tile_cfg=10)


@pytest.mark.parametrize('tile_cfg', [1, 2])
@pytest.mark.parametrize('K', [128, 640])
@pytest.mark.parametrize('dtype,blocks', [(torch.float16, (32, 32, 32)), (torch.bfloat16, (64, 32, 64)),
                                          (torch.float32, (16, 32, 16)), (torch.float16, (16, 32, 64)),
                                          (torch.float32, (64, 32, 32)), (torch.float16, (64, 32, 16)),
                                          (torch.float32, (32, 32, 32))])
@pytest.mark.parametrize('tA,tB', [(False, True), (True, False)])
def test_matmul_dds_tile_configs(tile_cfg, K, dtype, blocks, tA, tB, gpu):
    """Both sparse-output kernels (single-buffer and pipelined) on operands stored the same
    way round (k-contiguous, or [K, M] / [K, N] as in a weight gradient): stage counts
    below, equal to and above the depth of the register ring."""
    run_case(gpu, 'dds', tA, tB, True, True, dtype, blocks, batch=2, M=192, K=K, N=256,
             gran=(16, 16), sparsity=0.7, seed=5, tile_cfg=tile_cfg)


@pytest.mark.parametrize('tile_cfg', [0, 3, 4])
@pytest.mark.parametrize('compressed', [False, True])
@pytest.mark.parametrize('biased', [False, True])
@pytest.mark.parametrize('dtype,blocks,K', [(torch.float16, (64, 32, 64), 64), (torch.bfloat16, (32, 32, 64), 128),
                                            (torch.float32, (64, 32, 32), 32), (torch.float16, (32, 32, 32), 128),
                                            (torch.float32, (32, 32, 64), 64), (torch.bfloat16, (64, 32, 32), 64)])
def test_matmul_dds_block_row_kernel(tile_cfg, compressed, biased, dtype, blocks, K, gpu):
    """Sparse-output products whose whole K is one or two stages deep (attention scores):
    one workgroup walks the live blocks of a block row (tile config 3, or 4: a wavefront
    per 16 rows, 16-bit types and compressed output only); rows without a live block, one
    block and many."""
    if tile_cfg == 4 and (dtype == torch.float32 or not compressed):
        pytest.skip('tile config 4 takes 16-bit types and the compressed output layout')
    run_case(gpu, 'dds', False, True, biased, compressed, dtype, blocks, batch=3, M=448, K=K, N=320,
             gran=(32, 32), sparsity=0.8, seed=17, tile_cfg=tile_cfg)


@pytest.mark.parametrize('blocks', [(64, 32, 64), (32, 32, 32)])
def test_matmul_dds_block_rows_longer_than_a_wavefront(blocks, gpu):
    """Block rows with more than 64 live blocks (the column list no longer fits one
    register of a wavefront) and a batch that does not fill the eight-way numbering."""
    run_case(gpu, 'dds', False, True, False, True, torch.float16, blocks, batch=11, M=128, K=64, N=blocks[2] * 90,
             gran=(blocks[0], blocks[2]), sparsity=0.15, seed=23, tile_cfg=4)


@pytest.mark.parametrize('tile_cfg', [0, 9])
@pytest.mark.parametrize('compressed', [False, True])
@pytest.mark.parametrize('biased', [False, True])
@pytest.mark.parametrize('dtype,BK,N', [(torch.float16, 64, 64), (torch.bfloat16, 32, 64), (torch.float16, 32, 128),
                                        (torch.bfloat16, 64, 128)])
@pytest.mark.parametrize('tA', [False, True])
def test_matmul_thin_dense_operand(tile_cfg, compressed, biased, dtype, BK, N, tA, gpu):
    """Sparse first operand (as stored, or transposed as in the gradient of the second
    operand) times a [K, 64] / [K, 128] matrix - probabilities x values of an attention
    layer: the kernel with one workgroup per block row of the sparse operand; block rows
    without a live block, with one and with many; batch sizes that do not fill the
    eight-way workgroup numbering."""
    run_case(gpu, 'sdd', tA, False, biased, compressed, dtype, (64, BK, 32), batch=5, M=448, K=320, N=N,
             gran=(32, 32), sparsity=0.8, seed=19, tile_cfg=tile_cfg)


@pytest.mark.parametrize('tile_cfg', [0, 7])
@pytest.mark.parametrize('compressed', [False, True])
@pytest.mark.parametrize('mode,tA,tB', [('dsd', False, False), ('sdd', True, True), ('dsd', True, True), ('dsd', True, False),
                                        ('sdd', False, False), ('sdd', True, False)])
@pytest.mark.parametrize('dtype,blocks', [(torch.float16, (32, 32, 32)), (torch.bfloat16, (64, 64, 16)),
                                          (torch.float32, (16, 32, 64)), (torch.float16, (16, 64, 64))])
def test_matmul_panel_with_transposed_sparse_operand(tile_cfg, compressed, mode, tA, tB, dtype, blocks, gpu):
    """Every storage order of the two operands other than the all-k-contiguous one (the
    layouts of the backward kernels and of products with a [K, N] matrix), large and
    ragged enough for the panel kernel to be chosen and to clamp its last tile."""
    run_case(gpu, mode, tA, tB, True, compressed, dtype, blocks, batch=2,
             M=1096 if mode == 'dsd' else 128, K=128, N=128 if mode == 'dsd' else 1096, gran=(16, 16),
             sparsity=0.6, seed=13, tile_cfg=tile_cfg)


def test_matmul_all_ones_mask_is_plain_gemm(gpu):
    a_np, a = randn((1, 256, 128), 1, torch.float32)
    b_np, b = randn((1, 64, 128), 2, torch.float32)
    mask = torch.ones((64, 128), dtype=torch.uint8, device=gpu)
    kernel = SparTASparseMatMulKernel(mode='dsd', biased=False, transpose_A=False, transpose_B=True, compressed=False)
    kernel.ports['B'].set_mask(mask)
    kernel.set_shape(1, 256, 128, 64)
    kernel.compile({'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 32, 'BLOCK_SIZE_N_VALUE': 32})
    C = kernel(a.to(gpu), b.to(gpu))
    assert_close(C, a_np @ b_np.transpose(0, 2, 1), torch.float32)


def test_matmul_empty_mask_gives_zero_or_bias(gpu):
    _, a = randn((1, 128, 64), 1, torch.float16)
    _, b = randn((1, 64, 64), 2, torch.float16)
    bias_np, bias = randn((1, 64), 3, torch.float16)
    mask = torch.zeros((64, 64), dtype=torch.uint8, device=gpu)
    kernel = SparTASparseMatMulKernel(mode='dsd', biased=True, transpose_A=False, transpose_B=True, compressed=True)
    kernel.ports['B'].set_mask(mask)
    kernel.set_shape(1, 128, 64, 64)
    kernel.compile({'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 32, 'BLOCK_SIZE_N_VALUE': 32})
    w = kernel.ports['B'].indexes.convert(b.to(gpu))
    assert w.shape == (1, 0)
    C = kernel(a.to(gpu), w, bias.to(gpu))
    assert_close(C, np.broadcast_to(bias_np[:, None, :], (1, 128, 64)), torch.float16)


@pytest.mark.parametrize('tile_cfg', [0, 10])
def test_matmul_empty_mask_through_the_persistent_kernel(tile_cfg, gpu):
    """A fully pruned compressed weight at a shape that the dispatcher sends to the persistent
    kernel (tile config 10: batch 1, N / BN >= 128, M >= 4096, K / BK >= 32): the compressed
    operand is an empty tensor (a NULL pointer), every step of every tile is idle, and the
    output equals the bias."""
    M = K = N = 4096
    _, a = randn((1, M, K), 1, torch.float16)
    bias_np, bias = randn((1, N), 3, torch.float16)
    mask = torch.zeros((N, K), dtype=torch.uint8, device=gpu)
    kernel = SparTASparseMatMulKernel(mode='dsd', biased=True, transpose_A=False, transpose_B=True, compressed=True)
    kernel.ports['B'].set_mask(mask)
    kernel.set_shape(1, M, K, N)
    kernel.compile({'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 32, 'BLOCK_SIZE_N_VALUE': 32, 'TILE_CFG': tile_cfg})
    w = kernel.ports['B'].indexes.convert(torch.zeros((1, N, K), dtype=torch.float16, device=gpu))
    assert w.shape == (1, 0)
    C = kernel(a.to(gpu), w, bias.to(gpu))
    want = torch.from_numpy(bias_np).to(gpu).half().expand(M, N)
    assert torch.equal(C[0], want)


def test_matmul_ragged_m(gpu):
    """M that is not a multiple of the workgroup tile (dense dimension of 'dsd')."""
    for M in (16, 48, 200):
        run_case(gpu, 'dsd', False, True, True, True, torch.float16, (32, 32, 32), batch=1, M=M, K=128, N=64)


@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
def test_matmul_headline_shape_fp16(mode, gpu):
    """4096^3 fp16, 32x32 blocks at 95%: compared with a dense fp32 product of the
    masked operands computed on the GPU by torch (the CPU oracle takes minutes at
    this size; the small-shape tests above tie the kernels to the oracle)."""
    M = K = N = 4096
    g = torch.Generator().manual_seed(2022)
    A = torch.randn((1, M, K), generator=g).half().to(gpu)
    B = torch.randn((1, N, K), generator=g).half().to(gpu)
    mask_np = ops.block_mask((4096, 4096), (32, 32), 0.95, seed=2022)
    mask = torch.from_numpy(mask_np).to(gpu)
    kernel = SparTASparseMatMulKernel(mode=mode, biased=False, transpose_A=False, transpose_B=True, compressed=True)
    port = {'sdd': 'A', 'dsd': 'B', 'dds': 'C'}[mode]
    kernel.ports[port].set_mask(mask)
    kernel.set_shape(1, M, K, N)
    kernel.compile({'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 32, 'BLOCK_SIZE_N_VALUE': 32})
    idx = kernel.ports[port].indexes
    Af, Bf = A.float(), B.float()
    if mode == 'sdd':
        Af = Af * mask
        C = kernel(idx.convert(A * mask.half()), B)
    elif mode == 'dsd':
        Bf = Bf * mask
        C = kernel(A, idx.convert(B * mask.half()))
    else:
        C = idx.inverse(kernel(A, B))
    want = torch.matmul(Af, Bf.transpose(1, 2))
    if mode == 'dds':
        want = want * mask
    torch.testing.assert_close(C.float(), want, rtol=1e-2, atol=1e-2)


def _random_cases(n, seed):
    """Seeded draws over modes, layouts, dtypes, block shapes and ragged sizes: whatever
    kernel the dispatcher picks for each of them has to agree with the oracle."""
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        mode = ['sdd', 'dsd', 'dds'][rng.integers(3)]
        dtype = [torch.float16, torch.bfloat16, torch.float32][rng.integers(3)]
        blocks = tuple(int(x) for x in rng.choice([16, 32, 64], size=3))
        BM, BK, BN = blocks
        M = BM * int(rng.integers(1, 9)) * (4 if rng.random() < 0.3 else 1)
        K = BK * int(rng.integers(1, 7))
        N = BN * int(rng.integers(1, 9)) * (4 if rng.random() < 0.3 else 1)
        cases.append((mode, bool(rng.integers(2)), bool(rng.integers(2)), bool(rng.integers(2)), bool(rng.integers(2)),
                      dtype, blocks, int(rng.integers(1, 4)), M, K, N, float(rng.choice([0.0, 0.5, 0.8, 0.95])),
                      int(rng.integers(1 << 30))))
    return cases


@pytest.mark.parametrize('case', _random_cases(72, 2024), ids=lambda c: f'{c[0]}-{int(c[1])}{int(c[2])}{int(c[3])}{int(c[4])}-'
                         f'{str(c[5]).split(".")[-1]}-{c[6][0]}x{c[6][1]}x{c[6][2]}-{c[8]}x{c[9]}x{c[10]}')
def test_matmul_random_configurations(case, gpu):
    mode, tA, tB, biased, compressed, dtype, blocks, batch, M, K, N, sparsity, seed = case
    gran = tuple(int(g) for g in np.random.default_rng(seed).choice([4, 8, 16], size=2))
    run_case(gpu, mode, tA, tB, biased, compressed, dtype, blocks, batch=batch, M=M, K=K, N=N, gran=gran,
             sparsity=sparsity, seed=seed % 1000, tile_cfg=0)
