"""The benchmark configurations at their full sizes, through the operators, on the inputs
bench.py times:

  C3  SparseAttention, 96 heads x 4096 x 64 fp16, 64x64 blocks (causal window of 256
      tokens + 2% random blocks): the index bit-exact against the oracle, a sample of heads
      against the numpy oracle, every head fused vs the three-operator pipeline and vs a
      masked dense fp32 product on the GPU;
  C4  two SparseLinear(dynamic=True) layers 8192 x 768 -> 3072 -> 768 fp16 with a new top-10%
      mask of 32x64 blocks before every call: rebuilt index bit-exact against the oracle,
      output against the numpy oracle's masked-dense product, three mask updates, and the
      same step replayed from a HIP graph;
  C5  DynamicSparseMoE 16384 tokens, 1024 -> 4096, 8 experts, Zipf(1.2) routing: index
      bit-exact, output against the oracle's per-expert product;
  seqlen  SeqlenDynamicSparseAttention 32 x 12 x 1024 x 64 fp16, a sample of batch entries.
"""
import math

import numpy as np
import pytest
import torch

from oracle import bcs, ops
import sparta_amd as sparta
from helpers import assert_close

pytestmark = pytest.mark.gpu


# ------------------------------------------------------------------------------- C3
def attention_grid(n_blocks=64, seed=2022):
    grid = np.zeros((n_blocks, n_blocks), dtype=np.uint8)
    i, j = np.indices(grid.shape)
    grid[(i - j >= 0) & (i - j <= 4)] = 1
    grid |= (np.random.default_rng(seed).random(grid.shape) < 0.02).astype(np.uint8)
    return grid


def test_c3_attention_all_96_heads(gpu):
    BH, N, E, blk = 96, 4096, 64, 64
    grid = attention_grid()
    mask_np = np.kron(grid, np.ones((blk, blk), dtype=np.uint8))
    mask = torch.from_numpy(mask_np).to(gpu)
    g = torch.Generator().manual_seed(2022)
    q, k, v = (torch.randn((BH, N, E), generator=g).half() for _ in range(3))
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    att = sparta.nn.SparseAttention(mask=mask)
    mm = {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 64, 'BLOCK_SIZE_K_VALUE': 32, 'BLOCK_SIZE_N_VALUE': 64}
    att.build({'qk/forward:C': dict(mm),
               'sm/forward:y': {'_impl': 'sparta', 'BLOCK_SIZE_H_VALUE': 64, 'BLOCK_SIZE_W_VALUE': 64, 'ROW_TILE_VALUE': 4},
               'out/forward:C': {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 64, 'BLOCK_SIZE_K_VALUE': 64, 'BLOCK_SIZE_N_VALUE': 32}},
              sample_inputs=[qg, kg, vg])
    idx = att._sparse_port.indexes
    row_ptr, bcsr, nnz = bcs.build_bcsr(mask_np, blk, blk)
    assert idx.block_nnz == nnz == int(grid.sum())
    assert np.array_equal(idx.row_ptr.cpu().numpy(), row_ptr)
    assert np.array_equal(idx.BCSR_idx.cpu().numpy(), bcsr)
    with torch.no_grad():
        fused = att(qg, kg, vg)
        att._fused = False
        piped = att(qg, kg, vg)
        att._fused = True
    torch.testing.assert_close(fused.float(), piped.float(), rtol=1e-2, atol=1e-2)
    # every head against the masked dense product in fp32 on the GPU, twelve heads at a time
    live = mask.bool()
    for h0 in range(0, BH, 12):
        sl = slice(h0, h0 + 12)
        scores = torch.matmul(qg[sl].float(), kg[sl].float().transpose(1, 2)) / math.sqrt(E)
        scores.masked_fill_(~live, float('-inf'))
        want = torch.matmul(torch.softmax(scores, -1), vg[sl].float())
        torch.testing.assert_close(fused[sl].float(), want, rtol=1e-2, atol=1e-2)
    # heads from every residue of the eight-way workgroup numbering against the numpy oracle
    heads = [0, 1, 7, 8, 42, 95]
    qn, kn, vn = (t[heads].to(torch.float64).numpy() for t in (q, k, v))
    want = ops.attention_reference(qn, kn, vn, mask_np)
    assert_close(fused[heads], want, torch.float16, 'C3 fused attention, sampled heads')
    assert_close(piped[heads], want, torch.float16, 'C3 three-operator pipeline, sampled heads')


def _attention_train_config(bh, bw):
    mm = lambda m, k, n: {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': m, 'BLOCK_SIZE_K_VALUE': k, 'BLOCK_SIZE_N_VALUE': n}
    sm = {'_impl': 'sparta', 'BLOCK_SIZE_H_VALUE': bh, 'BLOCK_SIZE_W_VALUE': bw, 'ROW_TILE_VALUE': 4}
    return {'qk/forward:C': mm(bh, 32, bw), 'qk/backward:A': mm(bh, bw, 32), 'qk/backward:B': mm(bw, bh, 32),
            'sm/forward:y': dict(sm), 'sm/backward:x': dict(sm),
            'out/forward:C': mm(bh, bw, 32), 'out/backward:A': mm(bh, 32, bw), 'out/backward:B': mm(bw, bh, 32)}


@pytest.mark.parametrize('bh,bw', [(32, 32), (32, 64)])
def test_c3_training_step_with_other_block_shapes(bh, bw, gpu):
    """A well-formed SparseAttention training step at the full C3 size (96 heads x 4096 x 64
    fp16, the C3 mask) with score blocks other than 64x64, through its three paths - the
    kernels that recompute the probabilities, the kernels that store them, and the three
    operators with their six backward kernels - each against dense fp32 autograd on a sample of
    heads.  Every kernel of the step agrees on one block shape (build() refuses anything else)
    and every closure checks the size of its operands before it launches."""
    BH, N, E = 96, 4096, 64
    mask_np = np.kron(attention_grid(), np.ones((64, 64), dtype=np.uint8))
    mask = torch.from_numpy(mask_np).to(gpu)
    g = torch.Generator().manual_seed(2023)
    q, k, v, go = (torch.randn((BH, N, E), generator=g).half().to(gpu) for _ in range(4))
    heads = [0, 41, 95]
    # dense fp32 autograd on the sampled heads
    ref = [t[heads].float().requires_grad_(True) for t in (q, k, v)]
    scores = ref[0] @ ref[1].transpose(1, 2) / math.sqrt(E)
    scores = scores.masked_fill(mask == 0, float('-inf'))
    ref_out = torch.softmax(scores, -1) @ ref[2]
    ref_out.backward(go[heads].float())
    want = [ref_out.detach()] + [t.grad for t in ref]
    del scores

    for path, recompute, fused in (('recompute', True, True), ('stored probabilities', False, True),
                                   ('three operators', True, False)):
        print(f'C3 training step, blocks {bh}x{bw}, path: {path}', flush=True)
        att = sparta.nn.SparseAttention(mask=mask, recompute=recompute, fused=fused)
        leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
        att.build(_attention_train_config(bh, bw), sample_inputs=[t.detach() for t in leaves])
        idx = att._sparse_port.indexes
        assert (idx.block_H, idx.block_W) == (bh, bw)
        assert idx.block_nnz * bh * bw == int(attention_grid().sum()) * 64 * 64
        out = att(*leaves)
        out.backward(go)
        torch.cuda.synchronize()
        got = [out.detach()[heads].float()] + [t.grad[heads].float() for t in leaves]
        for name, a, b in zip(('out', 'grad_q', 'grad_k', 'grad_v'), got, want):
            torch.testing.assert_close(a, b, rtol=1e-2, atol=1e-2, msg=lambda m: f'{path}, {name}: {m}')
        del att, leaves, out, got


# ------------------------------------------------------------------------------- C4
def topk_block_mask(shape, seed, block=(32, 64), keep_frac=0.1):
    """Keeps the ceil(10%) blocks with the largest |score| (score ~ N(0,1), seeded)."""
    rows, cols = shape[0] // block[0], shape[1] // block[1]
    score = np.abs(np.random.default_rng(seed).standard_normal((rows, cols)))
    keep = math.ceil(keep_frac * rows * cols)
    thr = np.sort(score.ravel())[-keep]
    grid = (score >= thr).astype(np.uint8)
    return np.kron(grid, np.ones(block, dtype=np.uint8)), int(grid.sum())


@pytest.mark.parametrize('fused,batched', [(True, True), (True, False), (False, False)])
def test_c4_dynamic_ffn_three_mask_updates(fused, batched, gpu):
    # batched: both index rebuilds through sparta.nn.update_masks (one pair of launches), as bench.py issues them
    # fused: the activation between the layers runs in the first layer's epilogue (what bench.py times)
    act = (lambda h: h) if fused else torch.relu
    T, D, F = 8192, 768, 3072
    rng = np.random.default_rng(2022)
    x = torch.from_numpy(rng.standard_normal((T, D)).astype(np.float32)).half()
    w1 = torch.from_numpy((0.02 * rng.standard_normal((F, D))).astype(np.float32)).half()
    w2 = torch.from_numpy((0.02 * rng.standard_normal((D, F))).astype(np.float32)).half()
    l1 = torch.nn.Linear(D, F, bias=False, device=gpu, dtype=torch.float16)
    l2 = torch.nn.Linear(F, D, bias=False, device=gpu, dtype=torch.float16)
    with torch.no_grad():
        l1.weight.copy_(w1.to(gpu))
        l2.weight.copy_(w2.to(gpu))
    xg = x.to(gpu)
    masks1 = [topk_block_mask((F, D), s) for s in range(4)]
    masks2 = [topk_block_mask((D, F), 100 + s) for s in range(4)]
    assert all(n == 116 for _, n in masks1 + masks2)  # ceil(0.1 * 1152)
    cfg = {'forward:C': {'_impl': 'openai', 'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 64, 'BLOCK_SIZE_N_VALUE': 32}}
    op1 = sparta.nn.SparseLinear(l1, weight_mask=torch.from_numpy(masks1[0][0]).to(gpu), dynamic=True,
                                 activation='relu' if fused else None)
    op2 = sparta.nn.SparseLinear(l2, weight_mask=torch.from_numpy(masks2[0][0]).to(gpu), dynamic=True)
    with torch.no_grad():
        op1.build(cfg, sample_inputs=[xg])
        op2.build(cfg, sample_inputs=[act(op1(xg))])

    xn, w1n, w2n = (t.to(torch.float64).numpy() for t in (x, w1, w2))

    def oracle_step(m1, m2):
        h = ops.matmul_reference(xn[None], w1n[None], None, mode='dsd', transpose_A=False, transpose_B=True, mask=m1,
                                 dtype=np.float64)[0]
        h = np.maximum(h, 0.0)
        h16 = torch.from_numpy(h).half().to(torch.float64).numpy()  # the hidden activation is stored in fp16
        return ops.matmul_reference(h16[None], w2n[None], None, mode='dsd', transpose_A=False, transpose_B=True, mask=m2,
                                    dtype=np.float64)[0]

    for step in range(1, 4):  # three mask updates after the build
        m1, m2 = masks1[step][0], masks2[step][0]
        with torch.no_grad():
            if batched:
                sparta.nn.update_masks([(op1, {'weight_mask': torch.from_numpy(m1).to(gpu)}),
                                        (op2, {'weight_mask': torch.from_numpy(m2).to(gpu)})])
            else:
                op1.update_mask(weight_mask=torch.from_numpy(m1).to(gpu))
                op2.update_mask(weight_mask=torch.from_numpy(m2).to(gpu))
            y = op2(act(op1(xg)))
        for op, m in ((op1, m1), (op2, m2)):
            idx = op.get_sparse_indexes('B')
            row_ptr, bcsr, nnz = bcs.build_bcsr(m, 32, 64)
            assert idx.block_nnz == nnz == 116
            assert np.array_equal(idx.row_ptr.cpu().numpy(), row_ptr)
            assert np.array_equal(idx.BCSR_idx.cpu().numpy(), bcsr)
        assert_close(y, oracle_step(m1, m2), torch.float16, f'C4 dynamic FFN, mask update {step}')

    # the step bench.py times: both rebuilds and both products replayed from one HIP graph
    m1g = torch.from_numpy(masks1[0][0]).to(gpu).clone()
    m2g = torch.from_numpy(masks2[0][0]).to(gpu).clone()

    def graph_step():
        if batched:
            sparta.nn.update_masks([(op1, {'weight_mask': m1g}), (op2, {'weight_mask': m2g})])
        else:
            op1.update_mask(weight_mask=m1g)
            op2.update_mask(weight_mask=m2g)
        return op2(act(op1(xg)))

    with torch.no_grad():
        graph_step()
        torch.cuda.synchronize()
        stream = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            graph_step()
            stream.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                y_graph = graph_step()
        for replay in range(3):  # a new mask is copied into the captured buffers before every replay
            m1, m2 = masks1[replay + 1][0], masks2[replay + 1][0]
            m1g.copy_(torch.from_numpy(m1).to(gpu))
            m2g.copy_(torch.from_numpy(m2).to(gpu))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert_close(y_graph, oracle_step(m1, m2), torch.float16, f'C4 graph replay {replay}')


# ------------------------------------------------------------------------------- C5
def test_c5_moe_full_size(gpu):
    n_tok, n_exp, K, N = 16384, 8, 1024, 4096
    rng = np.random.default_rng(2022)
    w = torch.from_numpy((0.02 * rng.standard_normal((n_exp, N, K))).astype(np.float32)).half()
    mods = []
    for e in range(n_exp):
        lin = torch.nn.Linear(K, N, bias=False, dtype=torch.float16, device=gpu)
        with torch.no_grad():
            lin.weight.copy_(w[e].to(gpu))
        mods.append(lin)
    moe = sparta.nn.DynamicSparseMoE(mods)
    p = np.arange(1, n_exp + 1, dtype=np.float64) ** -1.2
    ids_np = np.random.default_rng(2022).choice(n_exp, size=n_tok, p=p / p.sum()).astype(np.int32)
    x = torch.from_numpy(rng.standard_normal((n_tok, K)).astype(np.float32)).half()
    with torch.no_grad():
        out = moe(x.to(gpu), torch.from_numpy(ids_np).to(gpu))
    count, offset, perm = ops.moe_index_reference(ids_np, n_exp)
    assert count.max() > 4096  # beyond the per-expert capacity the reference hard-codes (sparse_moe.py:23)
    assert np.array_equal(moe.expert_count.cpu().numpy(), count)
    assert np.array_equal(moe.expert_offset.cpu().numpy(), offset)
    assert np.array_equal(moe.sparse_index[:n_tok].cpu().numpy(), perm)
    weights_np = w.to(torch.float64).numpy().transpose(0, 2, 1)  # [E, in, out]
    want = ops.moe_reference(x.to(torch.float64).numpy(), weights_np, ids_np)
    assert_close(out, want, torch.float16, 'C5 MoE forward')


# --------------------------------------------------------------------------- seqlen
def test_seqlen_attention_benchmark_shape(gpu, B=32, H=12, N=1024, E=64):
    g = torch.Generator().manual_seed(2022)
    q, k, v = (torch.rand((B, H, N, E), generator=g).half() for _ in range(3))
    lens = np.random.default_rng(2022).integers(1, N, size=B).astype(np.int32)
    att = sparta.nn.SeqlenDynamicSparseAttention(global_mode=False)
    with torch.no_grad():
        out = att(q.to(gpu), k.to(gpu), v.to(gpu), torch.from_numpy(lens).to(gpu))
    # batch entries with the shortest, the longest and two other lengths; three heads each
    order = np.argsort(lens)
    for b in (int(order[0]), int(order[-1]), int(order[B // 2]), 5):
        L = int(lens[b])
        mask = np.zeros((N, N), dtype=np.uint8)
        mask[:L, :L] = 1
        heads = [0, 5, 11]
        qn, kn, vn = (t[b, heads].to(torch.float64).numpy() for t in (q, k, v))
        want = ops.attention_reference(qn, kn, vn, mask, temperature=1.0)
        assert_close(out[b, heads], want, torch.float16, f'seqlen attention b={b} L={L}')
        assert float(out[b, :, L:].abs().max()) == 0.0
