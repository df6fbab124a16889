"""GPU parity of SparseAttention against the numpy oracle: the three-operator
pipeline (fp32, as in the reference's test/unit/test_sparse_attention.py: 8x8
granular mask at 95%, atol 1e-4) and the fused forward kernel (fp16 / bf16,
element-granular and block-granular masks, mask updates)."""
import os

import numpy as np
import pytest
import torch

from oracle import ops
from sparta_amd.nn import SparseAttention
from helpers import randn, assert_close

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'vectors.npz'))


def config(bm, bk, bn, rt=4):
    mm = lambda: {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': bm, 'BLOCK_SIZE_K_VALUE': bk, 'BLOCK_SIZE_N_VALUE': bn}
    # qk: C tile (BM, BN); out: A tile (BM, BK) -> the shared tile is (bm, bn)
    out = {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': bm, 'BLOCK_SIZE_K_VALUE': bn, 'BLOCK_SIZE_N_VALUE': bk}
    return {'qk/forward:C': mm(), 'sm/forward:y': {'_impl': 'sparta', 'BLOCK_SIZE_H_VALUE': bm,
                                                    'BLOCK_SIZE_W_VALUE': bn, 'ROW_TILE_VALUE': rt},
            'out/forward:C': out}


@pytest.mark.parametrize('H', [1, 4])
@pytest.mark.parametrize('Nt,Ns,E', [(256, 256, 256), (512, 256, 64), (256, 512, 128)])
def test_attention_pipeline_fp32(H, Nt, Ns, E, gpu):
    q_np, q = randn((H, Nt, E), 1, torch.float32)
    k_np, k = randn((H, Ns, E), 2, torch.float32)
    v_np, v = randn((H, Ns, E), 3, torch.float32)
    att = None
    for seed in range(3):  # dynamic mask: update twice after the build
        mask_np = ops.block_mask((Nt, Ns), (8, 8), 0.95, seed=2022 + seed)
        mask = torch.from_numpy(mask_np).to(gpu)
        if att is None:
            att = SparseAttention(mask=mask)
            att.build(config(32, 32, 32), sample_inputs=[q.to(gpu), k.to(gpu), v.to(gpu)])
        else:
            att.update_mask(mask)
        out = att(q.to(gpu), k.to(gpu), v.to(gpu))  # fp32 runs the three-operator pipeline
        want = ops.attention_reference(q_np, k_np, v_np, mask_np)
        assert_close(out, want, torch.float32, f'attention fp32 seed {seed}')


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('blocks', [(64, 64), (32, 32), (16, 64), (64, 16), (32, 16)])
@pytest.mark.parametrize('gran', [(1, 1), (8, 8), None])
def test_attention_fused(dtype, blocks, gran, gpu, H=3, Nt=256, Ns=384, E=64):
    bm, bn = blocks
    q_np, q = randn((H, Nt, E), 4, dtype)
    k_np, k = randn((H, Ns, E), 5, dtype)
    v_np, v = randn((H, Ns, E), 6, dtype)
    mask_np = ops.block_mask((Nt, Ns), gran or blocks, 0.8 if gran else 0.6, seed=7)
    mask_np[40:48] = 0  # fully masked queries give zero rows
    att = SparseAttention(mask=torch.from_numpy(mask_np).to(gpu))
    att.build(config(bm, 32, bn), sample_inputs=[q.to(gpu), k.to(gpu), v.to(gpu)])
    with torch.no_grad():
        fused = att(q.to(gpu), k.to(gpu), v.to(gpu))
    want = ops.attention_reference(q_np, k_np, v_np, mask_np)
    assert_close(fused, want, dtype, f'fused attention {dtype} {blocks} {gran}')
    assert float(fused[:, 40:48].abs().max()) == 0.0
    # the pipeline (used when gradients are needed) agrees with the oracle as well
    qg = q.to(gpu).requires_grad_(True)
    piped = att(qg, k.to(gpu), v.to(gpu))
    assert piped.requires_grad
    assert_close(piped, want, dtype, 'pipelined attention')


@pytest.mark.parametrize('E', [32, 128])
def test_attention_fused_head_dims(E, gpu):
    q_np, q = randn((2, 128, E), 8, torch.float16)
    k_np, k = randn((2, 256, E), 9, torch.float16)
    v_np, v = randn((2, 256, E), 10, torch.float16)
    mask_np = ops.block_mask((128, 256), (32, 32), 0.5, seed=11)
    att = SparseAttention(mask=torch.from_numpy(mask_np).to(gpu))
    att.build(config(32, 32, 32), sample_inputs=[q.to(gpu), k.to(gpu), v.to(gpu)])
    with torch.no_grad():
        out = att(q.to(gpu), k.to(gpu), v.to(gpu))
    assert_close(out, ops.attention_reference(q_np, k_np, v_np, mask_np), torch.float16, f'E={E}')


def test_attention_golden_vectors(gpu):
    q, k, v = (torch.from_numpy(GOLD[n]).half().to(gpu) for n in ('att_q', 'att_k', 'att_v'))
    att = SparseAttention(mask=torch.from_numpy(GOLD['att_mask']).to(gpu))
    att.build(config(16, 32, 16), sample_inputs=[q, k, v])
    with torch.no_grad():
        assert_close(att(q, k, v), GOLD['att_out'], torch.float16, 'attention golden')


def test_attention_all_ones_mask_matches_sdpa(gpu):
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn((2, 128, 64), generator=g).half().to(gpu) for _ in range(3))
    att = SparseAttention(mask=torch.ones((128, 128), dtype=torch.uint8, device=gpu))
    att.build(config(64, 32, 64), sample_inputs=[q, k, v])
    with torch.no_grad():
        out = att(q, k, v)
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    torch.testing.assert_close(out.float(), want, rtol=1e-2, atol=1e-2)


def test_attention_long_sequence_layout(gpu):
    """Causal local window of 256 tokens plus 2% random blocks on a 64x64 block grid
    (4096 x 4096 mask), 4 heads of the full-size problem: fused vs the pipeline."""
    N, E, blk = 4096, 64, 64
    grid = np.zeros((64, 64), dtype=np.uint8)
    i, j = np.indices(grid.shape)
    grid[(i - j >= 0) & (i - j <= 4)] = 1
    grid |= (np.random.default_rng(2022).random(grid.shape) < 0.02).astype(np.uint8)
    mask = torch.from_numpy(np.kron(grid, np.ones((blk, blk), dtype=np.uint8))).to(gpu)
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn((4, N, E), generator=g).half().to(gpu) for _ in range(3))
    att = SparseAttention(mask=mask)
    att.build(config(64, 32, 64), sample_inputs=[q, k, v])
    assert att._sparse_port.indexes.block_nnz == int(grid.sum())
    with torch.no_grad():
        fused = att(q, k, v)
        att._fused = False
        piped = att(q, k, v)
    torch.testing.assert_close(fused.float(), piped.float(), rtol=1e-2, atol=1e-2)
    # first block-row attends to block 0 only (plus random extras): compare with dense torch
    live = torch.from_numpy(np.kron(grid[:1], np.ones((blk, blk), dtype=np.uint8))).to(gpu).bool()
    scores = (q[:, :blk].float() @ k.float().transpose(1, 2)) / 8.0
    scores = scores.masked_fill(~live, float('-inf'))
    want = torch.softmax(scores, -1) @ v.float()
    torch.testing.assert_close(fused[:, :blk].float(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('element_mask', [False, True])
@pytest.mark.parametrize('BH,BW,E', [(64, 64, 64), (32, 32, 64), (32, 128, 64), (64, 32, 128), (128, 64, 64),
                                     (128, 128, 128), (64, 128, 128), (32, 64, 128), (128, 32, 128)])
def test_attention_kernel_variants(dtype, element_mask, BH, BW, E, gpu):
    """The fused kernels through the C ABI (tile configs 1, 2 and 3) on the same inputs:
    each against the oracle, batch sizes that do not fill the eight-way workgroup
    numbering, empty block rows and (element_mask) partly filled blocks."""
    from sparta_amd import _lib
    from sparta_amd.tesa import get_bcs_function
    batch, Nt, Ns = 11, 2 * 128, 3 * 128
    q_np, q = randn((batch, Nt, E), 21, dtype)
    k_np, k = randn((batch, Ns, E), 22, dtype)
    v_np, v = randn((batch, Ns, E), 23, dtype)
    gran = (1, 1) if element_mask else (BH, BW)
    mask_np = ops.block_mask((Nt, Ns), gran, 0.7 if element_mask else 0.5, seed=24)
    mask_np[:BH] = 0  # an empty block row
    mask = torch.from_numpy(mask_np).to(gpu)
    indexes = get_bcs_function(BH, BW, True, False).build_indexes(mask)
    q, k, v = q.to(gpu), k.to(gpu), v.to(gpu)
    want = ops.attention_reference(q_np, k_np, v_np, mask_np)
    lib = _lib.load()
    for cfg in (1, 2, 3):
        out = torch.full_like(q, float('nan'))
        if cfg == 3 and not 1 <= (BW * E // 8) // (BH * 2) <= 8:
            continue  # the wide-MFMA kernel stages one to eight vectors per thread and tile
        rc = lib.spx_attention_forward(
            _lib.dtype_code(dtype), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v), _lib.dev_ptr(out),
            _lib.dev_ptr(indexes.row_ptr), _lib.dev_ptr(indexes._bcsr_buf),
            _lib.dev_ptr(indexes.raw_mask) if element_mask else None,
            1.0 / float(np.sqrt(E)), batch, Nt, Ns, E, BH, BW, cfg, _lib.current_stream(q.device))
        _lib.check(rc, 'spx_attention_forward')
        assert_close(out, want, dtype, f'attention tile config {cfg} {dtype} {(BH, BW, E)} mask={element_mask}')
        assert float(out[:, :BH].abs().max()) == 0.0


def train_config(bh, bw):
    mm = lambda m, k, n: {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': m, 'BLOCK_SIZE_K_VALUE': k, 'BLOCK_SIZE_N_VALUE': n}
    sm = {'_impl': 'sparta', 'BLOCK_SIZE_H_VALUE': bh, 'BLOCK_SIZE_W_VALUE': bw, 'ROW_TILE_VALUE': 4}
    # the score tile (bh, bw) is (BM, BN) of qk, (BM, BK) of out and of their backward kernels' sparse operands
    return {'qk/forward:C': mm(bh, 32, bw), 'qk/backward:A': mm(bh, bw, 32), 'qk/backward:B': mm(bw, bh, 32),
            'sm/forward:y': dict(sm), 'sm/backward:x': dict(sm),
            'out/forward:C': mm(bh, bw, 32), 'out/backward:A': mm(bh, 32, bw), 'out/backward:B': mm(bw, bh, 32)}


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('bh,bw,E', [(64, 64, 64), (32, 64, 64), (64, 32, 128), (64, 64, 128)])
@pytest.mark.parametrize('gran,recompute', [((1, 1), True), (None, False), (None, True)])
def test_attention_training_forward_kernel(dtype, bh, bw, E, gran, recompute, gpu, H=3, Nt=256, Ns=384):
    """With gradients recorded and the backward kernels built, the forward pass is one
    launch that also writes the probabilities - or, for a block-level mask with
    recompute=True, one number per query from which the two backward launches recompute
    them: output and the three gradients agree with the three-operator pipeline and with
    dense fp32 autograd; empty block rows and (with an element-granular mask) partly masked
    blocks and fully masked queries included."""
    _, q = randn((H, Nt, E), 31, dtype)
    _, k = randn((H, Ns, E), 32, dtype)
    _, v = randn((H, Ns, E), 33, dtype)
    _, g = randn((H, Nt, E), 34, dtype)
    mask_np = ops.block_mask((Nt, Ns), gran or (bh, bw), 0.8 if gran else 0.6, seed=35)
    mask_np[:bh] = 0            # an empty block row
    block_level = recompute and gran is None
    if not block_level:
        mask_np[bh + 3] = 0     # a fully masked query inside a live block row (the mask is then not block-level)
    mask = torch.from_numpy(mask_np).to(gpu)
    att = SparseAttention(mask=mask, recompute=recompute)
    leaves = [t.to(gpu).requires_grad_(True) for t in (q, k, v)]
    att.build(train_config(bh, bw), sample_inputs=[t.detach() for t in leaves])
    calls = []
    bwd_calls = []
    if block_level:   # no probabilities are stored
        inner = att._fused_forward_lse
        att._fused_forward_lse = lambda *a: (calls.append(1), inner(*a))[1]
        inner_bwd = att._recompute_backward_q
        att._recompute_backward_q = lambda *a: (bwd_calls.append(1), inner_bwd(*a))[1]
        inner_kv = att._recompute_backward_kv
        att._recompute_backward_kv = lambda *a: (bwd_calls.append(2), inner_kv(*a))[1]
        att._fused_forward_train = None
    else:
        inner = att._fused_forward_train
        att._fused_forward_train = lambda *a: (calls.append(1), inner(*a))[1]
        inner_bwd = att._fused_backward_scores
        att._fused_backward_scores = lambda *a, **kw: (bwd_calls.append(1), inner_bwd(*a, **kw))[1]
        inner_kv = att._fused_backward_kv
        att._fused_backward_kv = lambda *a: (bwd_calls.append(2), inner_kv(*a))[1]
        att._fused_forward_lse = None

    def run(fused):
        att._fused = fused
        for t in leaves:
            t.grad = None
        out = att(*leaves)
        out.backward(g.to(gpu))
        return [out.detach().float()] + [t.grad.detach().float() for t in leaves]

    got = run(True)
    assert calls, 'the training forward kernel was not used'
    piped = run(False)
    assert len(calls) == 1 and bwd_calls == [1, 2]
    # dense fp32 autograd on the same (rounded) inputs
    ref_leaves = [t.detach().float().requires_grad_(True) for t in leaves]
    scores = ref_leaves[0] @ ref_leaves[1].transpose(1, 2) / float(np.sqrt(E))
    scores = scores.masked_fill(mask == 0, float('-inf'))
    probs = torch.softmax(scores, -1).nan_to_num(0.0)
    ref_out = probs @ ref_leaves[2]
    ref_out.backward(g.to(gpu).float())
    want = [ref_out.detach()] + [t.grad for t in ref_leaves]
    for name, a, b, c in zip(('out', 'grad_q', 'grad_k', 'grad_v'), got, piped, want):
        torch.testing.assert_close(a, c, rtol=1e-2, atol=1e-2, msg=lambda m: f'{name} vs dense autograd: {m}')
        torch.testing.assert_close(a, b, rtol=1e-2, atol=1e-2, msg=lambda m: f'{name} vs pipeline: {m}')
    assert float(got[0][:, :bh].abs().max()) == 0.0 and (block_level or float(got[0][:, bh + 3].abs().max()) == 0.0)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('BH,BW,E', [(32, 32, 64), (32, 128, 64), (64, 64, 64), (64, 128, 128), (128, 64, 64),
                                     (128, 128, 128), (128, 32, 128), (32, 64, 128), (64, 128, 64), (32, 128, 128),
                                     (64, 32, 64), (128, 128, 64)])
@pytest.mark.parametrize('element_mask', [False, True])
def test_attention_backward_scores_kernel(dtype, BH, BW, E, element_mask, gpu, batch=3, Nt=256, Ns=384):
    """spx_attention_forward_train followed by spx_attention_backward_scores through the
    C-ABI: the probabilities, the score gradient (expanded to dense) and the query gradient
    agree with dense fp32 autograd over every block shape the two kernels cover; an empty
    block row and, with an element mask, partly masked blocks included."""
    from sparta_amd import _lib
    from sparta_amd.tesa import get_bcs_function
    _, q = randn((batch, Nt, E), 41, dtype)
    _, k = randn((batch, Ns, E), 42, dtype)
    _, v = randn((batch, Ns, E), 43, dtype)
    _, g = randn((batch, Nt, E), 44, dtype)
    mask_np = ops.block_mask((Nt, Ns), (1, 1) if element_mask else (BH, BW), 0.8 if element_mask else 0.6, seed=45)
    mask_np[:BH] = 0
    mask = torch.from_numpy(mask_np).to(gpu)
    indexes = get_bcs_function(BH, BW, True, True).build_indexes(mask)
    q, k, v, g = q.to(gpu), k.to(gpu), v.to(gpu), g.to(gpu)
    inv_t = 1.0 / float(np.sqrt(E))
    lib = _lib.load()
    n_val = indexes.block_nnz * BH * BW
    out = torch.full_like(q, float('nan'))
    probs = torch.full((batch, n_val), float('nan'), dtype=dtype, device=gpu)
    rc = lib.spx_attention_forward_train(
        _lib.dtype_code(dtype), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v), _lib.dev_ptr(out),
        _lib.dev_ptr(probs), n_val, _lib.dev_ptr(indexes.row_ptr), _lib.dev_ptr(indexes._bcsr_buf),
        _lib.dev_ptr(indexes.raw_mask) if element_mask else None, inv_t, batch, Nt, Ns, E, BH, BW,
        _lib.current_stream(gpu))
    _lib.check(rc, 'spx_attention_forward_train')
    grad_scores = torch.full_like(probs, float('nan'))
    grad_q = torch.full_like(q, float('nan'))
    row_dot = torch.full((batch, Nt), float('nan'), dtype=torch.float32, device=gpu)
    rc = lib.spx_attention_backward_scores(
        _lib.dtype_code(dtype), _lib.dev_ptr(g), _lib.dev_ptr(out), _lib.dev_ptr(probs), _lib.dev_ptr(k), _lib.dev_ptr(v),
        _lib.dev_ptr(grad_scores), _lib.dev_ptr(grad_q), _lib.dev_ptr(row_dot), n_val, _lib.dev_ptr(indexes.row_ptr),
        _lib.dev_ptr(indexes._bcsr_buf), inv_t, batch, Nt, Ns, E, BH, BW, _lib.current_stream(gpu))
    _lib.check(rc, 'spx_attention_backward_scores')
    # without the score gradient: same grad_q
    grad_q2 = torch.full_like(q, float('nan'))
    rc = lib.spx_attention_backward_scores(
        _lib.dtype_code(dtype), _lib.dev_ptr(g), _lib.dev_ptr(out), _lib.dev_ptr(probs), _lib.dev_ptr(k), _lib.dev_ptr(v),
        None, _lib.dev_ptr(grad_q2), None, n_val, _lib.dev_ptr(indexes.row_ptr),
        _lib.dev_ptr(indexes._bcsr_buf), inv_t, batch, Nt, Ns, E, BH, BW, _lib.current_stream(gpu))
    _lib.check(rc, 'spx_attention_backward_scores')
    assert torch.equal(grad_q, grad_q2)

    qf, kf, vf = (t.float().requires_grad_(True) for t in (q, k, v))
    scores = (qf @ kf.transpose(1, 2)).requires_grad_(True)
    scores.retain_grad()
    masked = (scores * inv_t).masked_fill(mask == 0, float('-inf'))
    p_ref = torch.softmax(masked, -1).nan_to_num(0.0)
    (p_ref @ vf).backward(g.float())
    tol = dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(row_dot, (g.float() * out.float()).sum(-1) * inv_t, rtol=1e-3, atol=1e-3)
    if BH * E >= 32 * BW:
        grad_k = torch.full_like(k, float('nan'))
        grad_v = torch.full_like(v, float('nan'))
        rc = lib.spx_attention_backward_kv(
            _lib.dtype_code(dtype), _lib.dev_ptr(g), _lib.dev_ptr(q), _lib.dev_ptr(v), _lib.dev_ptr(probs),
            _lib.dev_ptr(row_dot), _lib.dev_ptr(grad_k), _lib.dev_ptr(grad_v), n_val, _lib.dev_ptr(indexes.col_ptr),
            _lib.dev_ptr(indexes._bcsc_buf), _lib.IDX_BCSC_I64, inv_t, batch, Nt, Ns, E, BH, BW, _lib.current_stream(gpu))
        _lib.check(rc, 'spx_attention_backward_kv')
        torch.testing.assert_close(grad_v.float(), vf.grad, **tol)
        torch.testing.assert_close(grad_k.float(), kf.grad, **tol)
    torch.testing.assert_close(indexes.inverse(probs).float(), p_ref.detach(), **tol)
    torch.testing.assert_close(indexes.inverse(grad_scores).float(), scores.grad, **tol)
    torch.testing.assert_close(grad_q.float(), qf.grad, **tol)
    assert float(grad_q[:, :BH].abs().max()) == 0.0


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('BH,BW,E', [(32, 32, 64), (32, 128, 64), (64, 64, 64), (64, 128, 128), (128, 64, 64),
                                     (128, 128, 128), (32, 64, 128), (64, 128, 64), (32, 128, 128),
                                     (64, 32, 64), (128, 128, 64), (64, 32, 128)])
def test_attention_recompute_kernels(dtype, BH, BW, E, gpu, batch=3, Nt=256, Ns=384):
    """spx_attention_forward_lse, spx_attention_backward_q and spx_attention_backward_kv_recompute
    through the C-ABI: output, the recorded log-sum-exp, the row constants and the three
    gradients agree with dense fp32 autograd over every block shape the kernels cover - no
    probabilities are stored anywhere; an empty block row, a block row with one live block
    and batch sizes that do not fill the eight-way workgroup numbering included."""
    from sparta_amd import _lib
    from sparta_amd.tesa import get_bcs_function
    _, q = randn((batch, Nt, E), 51, dtype)
    _, k = randn((batch, Ns, E), 52, dtype)
    _, v = randn((batch, Ns, E), 53, dtype)
    _, g = randn((batch, Nt, E), 54, dtype)
    mask_np = ops.block_mask((Nt, Ns), (BH, BW), 0.6, seed=55)
    mask_np[:BH] = 0
    if Nt >= 2 * BH:
        mask_np[BH:2 * BH] = 0
        mask_np[BH:2 * BH, :BW] = 1
    mask = torch.from_numpy(mask_np).to(gpu)
    indexes = get_bcs_function(BH, BW, True, True).build_indexes(mask)
    q, k, v, g = q.to(gpu), k.to(gpu), v.to(gpu), g.to(gpu)
    inv_t = 1.0 / float(np.sqrt(E))
    lib = _lib.load()
    st = _lib.current_stream(gpu)
    out = torch.full_like(q, float('nan'))
    lse = torch.full((batch, Nt), float('nan'), dtype=torch.float32, device=gpu)
    rc = lib.spx_attention_forward_lse(
        _lib.dtype_code(dtype), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v), _lib.dev_ptr(out), _lib.dev_ptr(lse),
        _lib.dev_ptr(indexes.row_ptr), _lib.dev_ptr(indexes._bcsr_buf), None, inv_t, batch, Nt, Ns, E, BH, BW, st)
    _lib.check(rc, 'spx_attention_forward_lse')
    grad_q = torch.full_like(q, float('nan'))
    row_dot = torch.full((batch, Nt), float('nan'), dtype=torch.float32, device=gpu)
    rc = lib.spx_attention_backward_q(
        _lib.dtype_code(dtype), _lib.dev_ptr(g), _lib.dev_ptr(out), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v),
        _lib.dev_ptr(lse), _lib.dev_ptr(grad_q), _lib.dev_ptr(row_dot), _lib.dev_ptr(indexes.row_ptr),
        _lib.dev_ptr(indexes._bcsr_buf), inv_t, batch, Nt, Ns, E, BH, BW, st)
    _lib.check(rc, 'spx_attention_backward_q')

    qf, kf, vf = (t.float().requires_grad_(True) for t in (q, k, v))
    masked = (qf @ kf.transpose(1, 2) * inv_t).masked_fill(mask == 0, float('-inf'))
    p_ref = torch.softmax(masked, -1).nan_to_num(0.0)
    o_ref = p_ref @ vf
    o_ref.backward(g.float())
    tol = dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(out.float(), o_ref.detach(), **tol)
    # natural-log log-sum-exp of the live scores = row_lse * ln 2; +inf where nothing is live
    lse_ref = torch.logsumexp(masked.detach(), -1)
    live = torch.isfinite(lse_ref)
    torch.testing.assert_close((lse * float(np.log(2.0)))[live], lse_ref[live], rtol=2e-3, atol=2e-3)
    assert bool(torch.isinf(lse[~live]).all()) and bool((lse[~live] > 0).all())
    torch.testing.assert_close(row_dot, (g.float() * out.float()).sum(-1) * inv_t, rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(grad_q.float(), qf.grad, **tol)
    assert float(grad_q[:, :BH].abs().max()) == 0.0
    if BH * E >= 32 * BW and BH <= 2 * BW:
        grad_k = torch.full_like(k, float('nan'))
        grad_v = torch.full_like(v, float('nan'))
        rc = lib.spx_attention_backward_kv_recompute(
            _lib.dtype_code(dtype), _lib.dev_ptr(g), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v), _lib.dev_ptr(lse),
            _lib.dev_ptr(row_dot), _lib.dev_ptr(grad_k), _lib.dev_ptr(grad_v), _lib.dev_ptr(indexes.col_ptr),
            _lib.dev_ptr(indexes._bcsc_buf), _lib.IDX_BCSC_I64, inv_t, batch, Nt, Ns, E, BH, BW, st)
        _lib.check(rc, 'spx_attention_backward_kv_recompute')
        torch.testing.assert_close(grad_v.float(), vf.grad, **tol)
        torch.testing.assert_close(grad_k.float(), kf.grad, **tol)
    else:
        rc = lib.spx_attention_backward_kv_recompute(
            _lib.dtype_code(dtype), _lib.dev_ptr(g), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(v), _lib.dev_ptr(lse),
            _lib.dev_ptr(row_dot), _lib.dev_ptr(q), _lib.dev_ptr(q), _lib.dev_ptr(indexes.col_ptr),
            _lib.dev_ptr(indexes._bcsc_buf), _lib.IDX_BCSC_I64, inv_t, batch, Nt, Ns, E, BH, BW, st)
        assert rc != 0 and 'BH <= 2 * BW' in _lib.last_error()


@pytest.mark.parametrize('needs', [(True, False, False), (False, True, False), (False, False, True), (True, False, True)])
def test_attention_training_partial_gradients(needs, gpu, H=2, Nt=256, Ns=256, E=64, bh=64, bw=64):
    """Only some of query / key / value require gradients: the fused backward returns exactly
    those, equal to dense fp32 autograd."""
    dtype = torch.float16
    _, q = randn((H, Nt, E), 51, dtype)
    _, k = randn((H, Ns, E), 52, dtype)
    _, v = randn((H, Ns, E), 53, dtype)
    _, g = randn((H, Nt, E), 54, dtype)
    mask_np = ops.block_mask((Nt, Ns), (bh, bw), 0.5, seed=55)
    mask_np[:, :bw] = 1
    mask = torch.from_numpy(mask_np).to(gpu)
    att = SparseAttention(mask=mask)
    leaves = [t.to(gpu).requires_grad_(n) for t, n in zip((q, k, v), needs)]
    att.build(train_config(bh, bw), sample_inputs=[t.detach() for t in leaves])
    out = att(*leaves)
    out.backward(g.to(gpu))
    ref = [t.detach().float().requires_grad_(n) for t, n in zip(leaves, needs)]
    scores = (ref[0] @ ref[1].transpose(1, 2) / float(np.sqrt(E))).masked_fill(mask == 0, float('-inf'))
    (torch.softmax(scores, -1) @ ref[2]).backward(g.to(gpu).float())
    for t, r, n in zip(leaves, ref, needs):
        if n:
            torch.testing.assert_close(t.grad.float(), r.grad, rtol=1e-2, atol=1e-2)
        else:
            assert t.grad is None


def test_attention_training_after_mask_update(gpu, H=3, Nt=256, Ns=256, E=64, bh=64, bw=64):
    """update_mask between training steps: the fused forward and both backward kernels follow
    the rebuilt index (BCSR and BCSC)."""
    dtype = torch.float16
    _, q = randn((H, Nt, E), 61, dtype)
    _, k = randn((H, Ns, E), 62, dtype)
    _, v = randn((H, Ns, E), 63, dtype)
    _, g = randn((H, Nt, E), 64, dtype)
    att = None
    for seed in range(3):
        mask_np = ops.block_mask((Nt, Ns), (bh, bw), 0.5, seed=70 + seed)
        mask_np[:bh, :bw] = 1
        mask = torch.from_numpy(mask_np).to(gpu)
        leaves = [t.to(gpu).requires_grad_(True) for t in (q, k, v)]
        if att is None:
            att = SparseAttention(mask=mask)
            att.build(train_config(bh, bw), sample_inputs=[t.detach() for t in leaves])
        else:
            att.update_mask(mask)
        out = att(*leaves)
        out.backward(g.to(gpu))
        ref = [t.detach().float().requires_grad_(True) for t in leaves]
        scores = (ref[0] @ ref[1].transpose(1, 2) / float(np.sqrt(E))).masked_fill(mask == 0, float('-inf'))
        ref_out = torch.softmax(scores, -1).nan_to_num(0.0) @ ref[2]
        ref_out.backward(g.to(gpu).float())
        torch.testing.assert_close(out.detach().float(), ref_out.detach(), rtol=1e-2, atol=1e-2)
        for t, r in zip(leaves, ref):
            torch.testing.assert_close(t.grad.float(), r.grad, rtol=1e-2, atol=1e-2)
