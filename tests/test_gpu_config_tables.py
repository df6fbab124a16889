"""The tuned-configuration tables shipped in sparta_amd/params/ on the GPU: every row is
built into an operator at a small shape and checked, forward and backward, against the
numpy oracle (a row that names a tile the kernels do not take fails here), and one point
of the sparsity x granularity sweep runs end to end with its correctness assertions
(the reference's bench checks every point the same way, test/bench/matmul/matmul.py:30-36)."""
import argparse
import os
import sys

import numpy as np
import pytest
import torch

from oracle import ops
import sparta_amd as sparta
from sparta_amd.common import config_table as ct
from helpers import randn, assert_close

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def table_rows(op):
    return ct.load_config_table(ct.packaged_table_dir(op), device_name='no such device')


def row_id(row):
    return f"g{row['granularity']}-s{row['sparsity']}"


@pytest.mark.parametrize('row', table_rows('matmul'), ids=row_id)
def test_matmul_table_row_builds_and_matches_oracle(row, gpu, M=256, K=192, N=320):
    """Shapes are multiples of every block edge of the search space (16, 32, 64)."""
    config = ct.unflatten_config(row)
    g = int(float(row['granularity']))
    a_np, a = randn((1, M, K), 1, torch.float16)
    b_np, b = randn((1, N, K), 2, torch.float16)
    gc_np, gc = randn((1, M, N), 3, torch.float16)
    mask_np = ops.block_mask((N, K), (g, g), 0.7, seed=4)
    mask = torch.from_numpy(mask_np).to(gpu)
    op = sparta.nn.SparseBatchMatMul(B_mask=mask, transpose_A=False, transpose_B=True, compressed=True)
    ag = a.to(gpu).requires_grad_(True)
    op.build(config, sample_inputs=[ag.detach(), b.to(gpu)])
    indexes = op.get_sparse_indexes('B')
    bc = indexes.convert(b.to(gpu)).requires_grad_(True)
    out = op(ag, bc)
    out.backward(gc.to(gpu))
    # forward: B is read through the index, i.e. masked at the block level of the row's tile
    live = indexes.get_mask().cpu().numpy()
    want = ops.matmul_reference(a_np, b_np, None, mode='dsd', transpose_A=False, transpose_B=True, mask=live,
                                dtype=np.float64)
    assert_close(out, want, torch.float16, f'forward, row {row_id(row)}')
    grad_a = gc_np @ (b_np * live)
    grad_b = np.swapaxes(gc_np, 1, 2) @ a_np
    assert_close(ag.grad, grad_a, torch.float16, f'grad A, row {row_id(row)}', scale=float(np.abs(grad_a).max()))
    assert_close(indexes.inverse(bc.grad), grad_b * live, torch.float16, f'grad B, row {row_id(row)}',
                 scale=float(np.abs(grad_b).max()))


@pytest.mark.parametrize('row', table_rows('attention'), ids=row_id)
def test_attention_table_row_builds_and_matches_oracle(row, gpu, H=2, Nt=256, Ns=320, E=64):
    config = ct.unflatten_config(row)
    g = int(float(row['granularity']))
    q_np, q = randn((H, Nt, E), 5, torch.float16)
    k_np, k = randn((H, Ns, E), 6, torch.float16)
    v_np, v = randn((H, Ns, E), 7, torch.float16)
    mask_np = ops.block_mask((Nt, Ns), (g, g), 0.7, seed=8)
    att = sparta.nn.SparseAttention(mask=torch.from_numpy(mask_np).to(gpu))
    leaves = [t.to(gpu).requires_grad_(True) for t in (q, k, v)]
    att.build(config, sample_inputs=[t.detach() for t in leaves])
    want = ops.attention_reference(q_np, k_np, v_np, mask_np)
    with torch.no_grad():
        assert_close(att(*[t.detach() for t in leaves]), want, torch.float16, f'forward, row {row_id(row)}')
    out = att(*leaves)
    assert_close(out, want, torch.float16, f'forward with gradients, row {row_id(row)}')
    # gradients against the masked dense computation in float64 (torch autograd on the CPU)
    g_np, grad = randn((H, Nt, E), 9, torch.float16)
    out.backward(grad.to(gpu))
    ref = [torch.from_numpy(x).requires_grad_(True) for x in (q_np, k_np, v_np)]
    scores = ref[0] @ ref[1].transpose(1, 2) / np.sqrt(E)
    scores = scores.masked_fill(torch.from_numpy(mask_np == 0), float('-inf'))
    probs = torch.softmax(scores, -1).nan_to_num(0.0)
    (probs @ ref[2]).backward(torch.from_numpy(g_np))
    for name, leaf, r in zip('qkv', leaves, ref):
        wantg = r.grad.numpy()
        assert_close(leaf.grad, wantg, torch.float16, f'grad {name}, row {row_id(row)}',
                     scale=max(float(np.abs(wantg).max()), 1.0))


@pytest.mark.parametrize('op_name', ['matmul', 'attention'])
def test_one_sweep_point_runs_with_its_assertions(op_name, gpu):
    """bench_sweep.py at one (granularity, sparsity) point with a short timing loop: the
    packaged row is looked up and built, output and gradients are asserted, and the
    latencies of the dense and the sparse method come back finite and positive."""
    if ROOT not in sys.path:
        sys.path.insert(0, ROOT)
    import bench_sweep
    args = argparse.Namespace(op=op_name, dtype='fp16', quick=True, tune=0, algo='rand', warmups=2, iters=3,
                              granularity=32, sparsity=0.95)
    sweep = bench_sweep.sweep_matmul if op_name == 'matmul' else bench_sweep.sweep_attention
    header, rows, tuned = sweep(args, torch, sparta, ct.packaged_table_dir(op_name), 'no such device')
    assert header[0] == 'method' and header[-2:] == ['forward', 'backward']
    assert [r[0] for r in rows] == ['dense', 'sparta_amd'] and not tuned
    for r in rows:
        assert all(np.isfinite(x) and x > 0 for x in r[-2:]), r
