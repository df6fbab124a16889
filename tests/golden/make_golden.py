"""Writes tests/golden/vectors.npz: small seeded input/output vectors for the
hot path, produced by the numpy oracle (oracle/), so that the GPU tests and the
CPU tests of the oracle both have fixed data to compare with.  The reference
keeps no stored vectors for this path (its tests recompute dense targets on a
CUDA device), so these are the repository's own fixtures.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import bcs, ops  # noqa: E402


def main():
    out = {}
    # index build: (H, W, BH, BW, granularity, sparsity, seed)
    cases = [(64, 96, 16, 32, (8, 8), 0.7, 1), (128, 128, 32, 32, (1, 1), 0.99, 2),
             (96, 64, 4, 8, (4, 4), 0.5, 3), (256, 256, 64, 64, (64, 64), 0.9, 4)]
    for i, (H, W, BH, BW, gran, sp, seed) in enumerate(cases):
        mask = ops.block_mask((H, W), gran, sp, seed)
        row_ptr, bcsr, col_ptr, bcsc64, nnz = bcs.build_bcsrc(mask, BH, BW)
        _, bcsc32, _ = bcs.build_bcsc(mask, BH, BW)
        out[f'idx{i}_meta'] = np.array([H, W, BH, BW, nnz])
        out[f'idx{i}_mask'] = mask
        out[f'idx{i}_row_ptr'] = row_ptr
        out[f'idx{i}_bcsr'] = bcsr
        out[f'idx{i}_col_ptr'] = col_ptr
        out[f'idx{i}_bcsc32'] = bcsc32
        out[f'idx{i}_bcsc64'] = bcsc64

    rng = np.random.default_rng(2022)
    # matmul: batch 2, M=64, K=96, N=32, blocks 32/32/32 (fp16-representable inputs)
    M, K, N = 64, 96, 32
    for mode in ('sdd', 'dsd', 'dds'):
        A = rng.standard_normal((2, M, K)).astype(np.float16).astype(np.float32)
        B = rng.standard_normal((2, N, K)).astype(np.float16).astype(np.float32)
        bias = rng.standard_normal((2, N)).astype(np.float16).astype(np.float32)
        shape = {'sdd': (M, K), 'dsd': (N, K), 'dds': (M, N)}[mode]
        mask = ops.block_mask(shape, (16, 16), 0.6, seed=7)
        C = ops.matmul_reference(A, B, bias, mode=mode, transpose_A=False, transpose_B=True, mask=mask,
                                 block=(32, 32), dtype=np.float64)
        out[f'mm_{mode}_A'], out[f'mm_{mode}_B'], out[f'mm_{mode}_bias'] = A, B, bias
        out[f'mm_{mode}_mask'], out[f'mm_{mode}_C'] = mask, C

    # softmax: batch 2, 32 x 64, temperature 8
    x = (rng.standard_normal((2, 32, 64)) * 3).astype(np.float16).astype(np.float32)
    g = rng.standard_normal((2, 32, 64)).astype(np.float16).astype(np.float32)
    mask = ops.block_mask((32, 64), (4, 4), 0.7, seed=9)
    mask[8:12] = 0
    y = ops.softmax_forward_reference(x, mask, 8.0)
    out['sm_x'], out['sm_g'], out['sm_mask'], out['sm_y'] = x, g, mask, y
    out['sm_gx'] = ops.softmax_backward_reference(g, y, mask, 8.0)

    # attention: 3 heads, 64 x 64, E = 32
    q, k, v = (rng.standard_normal((3, 64, 32)).astype(np.float16).astype(np.float32) for _ in range(3))
    mask = ops.block_mask((64, 64), (16, 16), 0.5, seed=11)
    out['att_q'], out['att_k'], out['att_v'], out['att_mask'] = q, k, v, mask
    out['att_out'] = ops.attention_reference(q, k, v, mask)

    # moe: 96 tokens, 4 experts, 64 -> 48
    tokens = rng.standard_normal((96, 64)).astype(np.float16).astype(np.float32)
    weights = (rng.standard_normal((4, 64, 48)) * 0.1).astype(np.float16).astype(np.float32)
    ids = rng.integers(0, 4, 96).astype(np.int32)
    out['moe_tokens'], out['moe_weights'], out['moe_ids'] = tokens, weights, ids
    out['moe_out'] = ops.moe_reference(tokens, weights, ids)
    count, offset, perm = ops.moe_index_reference(ids, 4)
    out['moe_count'], out['moe_offset'], out['moe_perm'] = count, offset, perm

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'vectors.npz')
    np.savez_compressed(path, **out)
    print(f'wrote {path} ({os.path.getsize(path)} bytes, {len(out)} arrays)')


if __name__ == '__main__':
    main()
