"""Host-side model of what the kernels of a SparseAttention training step walk behind their
pointers, at the full size of the attention benchmark (96 heads x 4096 x 4096 positions, 64x64
granular mask), and the checks that refuse a mis-sized operand before any launch.  No GPU: the
indexes come from the numpy oracle and the tensors are `meta` tensors (only numel() is read).

The case modelled: kernels that share one sparse tensor share one index object, which is
rebuilt for the block shape of whichever kernel was bound last.  A kernel bound earlier with
block shape X keeps the index of X - nnz_X blocks of X[0] x X[1] elements - and strides the
batch by nnz_X * X[0] * X[1], while the compressed tensor it is handed was laid out for the
last shape Y: [batch, nnz_Y * Y[0] * Y[1]].  Whenever X covers more area than Y the kernel
walks past the end of the allocation.
"""
import itertools

import numpy as np
import pytest
import torch

from oracle import bcs
from sparta_amd.specializer.kernels.operand_sizes import (
    attention_extent, check_matmul_operands, matmul_extent, require_numel, softmax_extent)

BATCH, N, E = 96, 4096, 64
SHAPES = [(32, 32), (32, 64), (64, 32), (64, 64), (32, 128), (128, 32), (64, 128), (128, 64), (128, 128)]


def attention_grid(n_blocks=64, seed=2022):
    """Block mask of the attention benchmark: causal window of five 64-blocks + 2 % random."""
    grid = np.zeros((n_blocks, n_blocks), dtype=np.uint8)
    i, j = np.indices(grid.shape)
    grid[(i - j >= 0) & (i - j <= 4)] = 1
    grid |= (np.random.default_rng(seed).random(grid.shape) < 0.02).astype(np.uint8)
    return grid


@pytest.fixture(scope='module')
def live_blocks():
    """{block shape: live block count} of the benchmark mask, from the oracle's index builder."""
    mask = np.kron(attention_grid(), np.ones((64, 64), dtype=np.uint8))
    return {shape: bcs.build_bcsr(mask, *shape)[2] for shape in SHAPES}


def _meta(*shape):
    return torch.empty(shape, dtype=torch.float16, device='meta')


def test_a_stale_block_shape_walks_past_the_compressed_tensor(live_blocks):
    """Elements per batch entry that a kernel bound to X walks, against the tensor laid out for
    Y.  Shapes that tile the 64x64 granularity cover exactly the live area; every coarser X
    covers more, so paired with any finer Y it over-reads - by up to hundreds of MB at 96 heads."""
    area = {shape: nnz * shape[0] * shape[1] for shape, nnz in live_blocks.items()}
    exact = int(attention_grid().sum()) * 64 * 64
    worst = 0
    for X, Y in itertools.permutations(SHAPES, 2):
        fine = lambda s: s[0] <= 64 and s[1] <= 64
        if fine(X):
            assert area[X] == exact
        else:
            assert area[X] > exact
        walked, held = BATCH * area[X], BATCH * area[Y]
        if fine(Y) and not fine(X):
            assert walked > held
            worst = max(worst, (walked - held) * 2)   # bytes of fp16 past the end
    # fp16: the tensor holds 307 MB; 128-wide or 128-high blocks walk 420 MB, 128x128 blocks
    # 547 MB - up to 240 MB past the end of the allocation
    assert BATCH * exact * 2 == 307_494_912
    assert BATCH * area[(128, 64)] * 2 == BATCH * area[(32, 128)] * 2 == 419_954_688
    assert worst == BATCH * area[(128, 128)] * 2 - 307_494_912 == 239_861_760


@pytest.mark.parametrize('X,Y', [(x, y) for x, y in itertools.permutations(SHAPES, 2)])
def test_every_closure_refuses_a_tensor_of_another_layout(live_blocks, X, Y):
    """The operand checks of the launch closures (AssertionError before the library is
    called) for the kernels of the training step, each bound to X and handed tensors of Y."""
    stride_x = live_blocks[X] * X[0] * X[1]
    stride_y = live_blocks[Y] * Y[0] * Y[1]
    scores_y = _meta(BATCH, stride_y)
    q, k = _meta(BATCH, N, E), _meta(BATCH, N, E)
    cases = [
        # P V and its gradients read the compressed probabilities as operand A
        lambda: check_matmul_operands(matmul_extent('sdd', True, BATCH, N, N, E, stride_x), scores_y, k, None, False),
        # gradient of q / k from the compressed score gradient
        lambda: check_matmul_operands(matmul_extent('sdd', True, BATCH, N, N, E, stride_x), scores_y, q, None, False),
        # softmax forward / backward over the compressed scores
        lambda: require_numel('spx_softmax_forward', 'x', scores_y, softmax_extent(True, BATCH, N, N, stride_x)),
        # the fused backward kernels read the saved probabilities
        lambda: require_numel('spx_attention_backward_scores', 'probs', scores_y,
                              attention_extent(BATCH, N, N, E, live_blocks[X], *X).probs),
    ]
    for case in cases:
        if stride_x == stride_y:
            case()   # same extent: nothing is read out of bounds (build() still refuses the mix)
        else:
            with pytest.raises(AssertionError):
                case()


@pytest.mark.parametrize('shape', SHAPES)
def test_well_formed_training_step_stays_inside_its_tensors(live_blocks, shape):
    """Every kernel of a well-formed step (all kernels on one block shape) against the tensors
    the operators allocate for it: the bounds the full-size GPU test relies on."""
    nnz = live_blocks[shape]
    stride = nnz * shape[0] * shape[1]
    want = attention_extent(BATCH, N, N, E, nnz, *shape)
    assert want.probs == BATCH * stride and want.q == want.kv == BATCH * N * E and want.rows == BATCH * N
    q, k, v, out = (_meta(BATCH, N, E) for _ in range(4))
    scores = _meta(BATCH, stride)
    # q k^T -> compressed scores (C), softmax, P v
    ext = matmul_extent('dds', True, BATCH, N, E, N, stride)
    check_matmul_operands(ext, q, k, None, False)
    assert ext.C == scores.numel()
    require_numel('spx_softmax_forward', 'x', scores, softmax_extent(True, BATCH, N, N, stride))
    ext = matmul_extent('sdd', True, BATCH, N, N, E, stride)
    check_matmul_operands(ext, scores, v, None, False)
    assert ext.C == out.numel()
    # index entries address whole blocks inside the mask: (block_row + 1) * BH <= N
    mask = np.kron(attention_grid(), np.ones((64, 64), dtype=np.uint8))
    _, idx, _ = bcs.build_bcsr(mask, *shape)
    assert ((idx >> 16) + 1).max() * shape[0] <= N and ((idx & 0xffff) + 1).max() * shape[1] <= N


def test_dense_operands_are_checked_too():
    ext = matmul_extent('dsd', True, 1, 4096, 4096, 4096, 848 * 1024)
    x, w = _meta(4096, 4096), _meta(848 * 1024)
    check_matmul_operands(ext, x, w, _meta(4096), True)
    with pytest.raises(AssertionError, match='A has'):
        check_matmul_operands(ext, _meta(2048, 4096), w, _meta(4096), True)
    with pytest.raises(AssertionError, match='bias is required'):
        check_matmul_operands(ext, x, w, None, True)
    with pytest.raises(AssertionError, match='B has'):
        check_matmul_operands(ext, x, _meta(819 * 1024), None, False)
