"""GPU tests of the operator layer (the drop-in API): SparseLinear with each mask
kind, tune() / build(), mask updates, autograd through the sparse kernels, the
README flow of the reference, and the host-sync-free dynamic mode.  Targets are
the numpy oracle or dense torch autograd on the masked operands, as in the
reference's test/unit/test_sparse_matmul.py:177-339 and test_sparse_softmax.py."""
import numpy as np
import pytest
import torch

import sparta_amd as sparta
from oracle import ops
from helpers import randn, rand, assert_close

pytestmark = pytest.mark.gpu

CFG32 = {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 32, 'BLOCK_SIZE_N_VALUE': 32}


def dense_linear(K, N, w, b, gpu, dtype=torch.float32):
    lin = torch.nn.Linear(K, N, bias=b is not None, device=gpu, dtype=dtype)
    with torch.no_grad():
        lin.weight.copy_(w.to(gpu))
        if b is not None:
            lin.bias.copy_(b.to(gpu))
    return lin


def test_readme_flow_fp32(gpu):
    """README case: 1024^3 fp32, 8x8-granular 90% weight mask, tune(rand), compare
    with the masked dense linear (tolerance 1e-4)."""
    M = K = N = 1024
    x_np, x = rand((M, K), 1)
    w_np, w = rand((N, K), 2)
    b_np, b = rand((N,), 3)
    mask_np = ops.block_mask((N, K), (8, 8), 0.9, seed=2022)
    mask = torch.from_numpy(mask_np).to(gpu)
    lin = dense_linear(K, N, w * torch.from_numpy(mask_np), b, gpu)
    op = sparta.nn.SparseLinear(lin, weight_mask=mask)
    best = sparta.nn.tune(op, sample_inputs=[x.to(gpu)], max_trials=10, algo='rand')
    assert set(best) == {'root'} and best['root']['forward:C']['_impl'] in ('sparta', 'openai')
    assert op.ready and op.weight.dim() == 1
    y = op(x.to(gpu))
    want = ops.matmul_reference(x_np[None], w_np[None], b_np[None], mode='dsd', transpose_A=False,
                                transpose_B=True, mask=mask_np, dtype=np.float64)[0]
    g, wnt = y.detach().double().cpu().numpy(), want
    assert np.all(np.abs(g - wnt) <= 1e-4 + 1e-4 * np.abs(wnt)), np.abs(g - wnt).max()


@pytest.mark.parametrize('kind', ['input', 'weight'])
@pytest.mark.parametrize('dtype', [torch.float32, torch.float16])
@pytest.mark.parametrize('dynamic', [False, True])
def test_sparse_linear_fused_relu(kind, dtype, dynamic, gpu, M=128, K=256, N=192):
    """SparseLinear(activation='relu'): relu(x W^T + b) from the matmul kernel's epilogue, with
    the gradients of relu(linear) (the incoming gradient is gated by the sign of the output)."""
    x_np, x = randn((M, K), 14, dtype)
    w_np, w = randn((N, K), 15, dtype, scale=0.5)
    b_np, b = randn((N,), 16, dtype)
    gy_np, gy = randn((M, N), 17, dtype)
    shape = {'input': (M, K), 'weight': (N, K)}[kind]
    mask_np = ops.block_mask(shape, (8, 8), 0.9, seed=3)
    mask = torch.from_numpy(mask_np).to(gpu)
    w_in = w * torch.from_numpy(mask_np).to(dtype) if kind == 'weight' else w
    op = sparta.nn.SparseLinear(dense_linear(K, N, w_in, b, gpu, dtype), dynamic=dynamic, activation='relu',
                                **{f'{kind}_mask': mask})
    cfg = {k: dict(CFG32) for k in ('forward:C', 'backward:A', 'backward:B')}
    op.build(cfg, sample_inputs=[x.to(gpu)])
    xr = (x.to(gpu).float() * (mask if kind == 'input' else 1)).requires_grad_(True)
    wr = (w.to(gpu).float() * (mask if kind == 'weight' else 1)).requires_grad_(True)
    br = b.to(gpu).float().requires_grad_(True)
    pre = torch.nn.functional.linear(xr, wr, br)
    xs = (x.to(gpu) * (mask.to(dtype) if kind == 'input' else 1)).requires_grad_(True)
    y = op(xs)
    assert float(y.detach().min()) >= 0.0
    assert_close(y, torch.relu(pre).detach().double().cpu().numpy(), dtype, f'{kind} relu forward')
    y.backward(gy.to(gpu))
    # the reference gradient is gated by the operator's own output: an entry within rounding
    # of zero may fall on either side, and either gate is a correct derivative there
    pre.backward(gy.to(gpu).float() * (y.detach() > 0))
    block_mask = op.get_sparse_indexes({'input': 'A', 'weight': 'B'}[kind]).get_mask()
    gx_want = xr.grad * (block_mask if kind == 'input' else 1)
    assert_close(xs.grad, gx_want.double().cpu().numpy(), dtype, f'{kind} relu grad_x')
    gw = op.weight.grad
    if kind == 'weight' and not dynamic:
        gw = op.get_sparse_indexes('B').inverse(gw)
    gw_want = wr.grad * (block_mask if kind == 'weight' else 1)
    assert_close(gw if kind == 'input' else gw * block_mask.to(gw.dtype), gw_want.double().cpu().numpy(), dtype, f'{kind} relu grad_w')
    assert_close(op.bias.grad, br.grad.double().cpu().numpy(), dtype, f'{kind} relu grad_b')
    with pytest.raises(ValueError):
        sparta.nn.SparseLinear(dense_linear(K, N, w, b, gpu, dtype), output_mask=torch.ones((M, N), device=gpu), activation='relu')
    with pytest.raises(ValueError):
        sparta.nn.SparseLinear(dense_linear(K, N, w_in, b, gpu, dtype), weight_mask=mask, activation='gelu')


@pytest.mark.parametrize('kind', ['input', 'weight', 'output'])
@pytest.mark.parametrize('dtype', [torch.float32, torch.float16])
def test_sparse_linear_forward_backward_and_mask_updates(kind, dtype, gpu, M=128, K=256, N=192):
    x_np, x = randn((M, K), 4, dtype)
    w_np, w = randn((N, K), 5, dtype, scale=0.5)
    b_np, b = randn((N,), 6, dtype)
    gy_np, gy = randn((M, N), 7, dtype)
    shape = {'input': (M, K), 'weight': (N, K), 'output': (M, N)}[kind]
    op = None
    for seed in range(3):
        mask_np = ops.block_mask(shape, (8, 8), 0.9, seed=seed)
        mask = torch.from_numpy(mask_np).to(gpu)
        # As in the reference, the weight is handed over already masked: values inside
        # live blocks are used as they are.
        w_in = w * torch.from_numpy(mask_np).to(dtype) if kind == 'weight' else w
        if op is None:
            op = sparta.nn.SparseLinear(dense_linear(K, N, w_in, b, gpu, dtype), **{f'{kind}_mask': mask})
            cfg = {k: dict(CFG32) for k in ('forward:C', 'backward:A', 'backward:B')}
            op.build(cfg, sample_inputs=[x.to(gpu)])
        else:
            op._raw_weight = w_in.to(gpu)
            op.update_mask(**{f'{kind}_mask': mask})
        # dense torch reference on the masked operands (autograd gives the gradients)
        xr = (x.to(gpu).float() * (mask if kind == 'input' else 1)).requires_grad_(True)
        wr = (w.to(gpu).float() * (mask if kind == 'weight' else 1)).requires_grad_(True)
        br = b.to(gpu).float().requires_grad_(True)
        block_mask = op.get_sparse_indexes({'input': 'A', 'weight': 'B', 'output': 'C'}[kind]).get_mask()
        yr = torch.nn.functional.linear(xr, wr, br)
        if kind == 'output':
            yr = yr * block_mask
        yr.backward(gy.to(gpu).float())

        xs = (x.to(gpu) * (mask.to(dtype) if kind == 'input' else 1)).requires_grad_(True)
        y = op(xs)
        assert_close(y, yr.detach().double().cpu().numpy(), dtype, f'{kind} forward')
        grad_in = gy.to(gpu) * (block_mask.to(dtype) if kind == 'output' else 1)
        y.backward(grad_in)
        gx_want = xr.grad * (block_mask if kind == 'input' else 1)  # masked inputs get no gradient
        assert_close(xs.grad, gx_want.double().cpu().numpy(), dtype, f'{kind} grad_x')
        gw = op.weight.grad
        if kind == 'weight':
            gw = op.get_sparse_indexes('B').inverse(gw)
            gw_want = wr.grad * block_mask
        else:
            gw_want = wr.grad
        assert_close(gw, gw_want.double().cpu().numpy(), dtype, f'{kind} grad_w')
        assert_close(op.bias.grad, br.grad.double().cpu().numpy(), dtype, f'{kind} grad_b')
        op.weight.grad = None
        op.bias.grad = None


@pytest.mark.parametrize('mode,tA,tB,compressed', [
    ('sdd', False, False, True), ('dsd', True, True, True), ('dds', False, True, True),
    ('dds', True, False, False), ('sdd', True, True, False),
])
def test_sparse_batch_matmul_operator(mode, tA, tB, compressed, gpu, Bt=3, M=128, K=192, N=64):
    a_np, a = randn((Bt, K, M) if tA else (Bt, M, K), 8)
    b_np, b = randn((Bt, N, K) if tB else (Bt, K, N), 9)
    g_np, g = randn((Bt, M, N), 10)
    port = {'sdd': 'A', 'dsd': 'B', 'dds': 'C'}[mode]
    shape = {'A': a.shape[1:], 'B': b.shape[1:], 'C': (M, N)}[port]
    mask_np = ops.block_mask(shape, (8, 8), 0.9, seed=11)
    mask = torch.from_numpy(mask_np).to(gpu)
    op = sparta.nn.SparseBatchMatMul(**{f'{port}_mask': mask}, transpose_A=tA, transpose_B=tB,
                                     compressed=compressed)
    cfg = {k: dict(CFG32) for k in ('forward:C', 'backward:A', 'backward:B')}
    op.build(cfg, sample_inputs=[a.to(gpu), b.to(gpu)])
    idx = op.get_sparse_indexes(port)
    block_mask = idx.get_mask()

    ar = (a.to(gpu) * (mask if port == 'A' else 1)).requires_grad_(True)
    br_ = (b.to(gpu) * (mask if port == 'B' else 1)).requires_grad_(True)
    cr = torch.matmul(ar.transpose(1, 2) if tA else ar, br_.transpose(1, 2) if tB else br_)
    if port == 'C':
        cr = cr * block_mask
    cr.backward(g.to(gpu))

    a_in = (a.to(gpu) * (mask if port == 'A' else 1))
    b_in = (b.to(gpu) * (mask if port == 'B' else 1))
    if compressed and port == 'A':
        a_in = idx.convert(a_in)
    if compressed and port == 'B':
        b_in = idx.convert(b_in)
    a_in.requires_grad_(True)
    b_in.requires_grad_(True)
    c = op(a_in, b_in)
    c_dense = idx.inverse(c) if (compressed and port == 'C') else c
    assert_close(c_dense, cr.detach().double().cpu().numpy(), torch.float32, 'forward')
    grad = g.to(gpu) * (block_mask if port == 'C' else 1)
    c.backward(idx.convert(grad) if (compressed and port == 'C') else grad)
    ga = idx.inverse(a_in.grad) if (compressed and port == 'A') else a_in.grad
    gb = idx.inverse(b_in.grad) if (compressed and port == 'B') else b_in.grad
    ga_want = ar.grad * (block_mask if port == 'A' else 1)
    gb_want = br_.grad * (block_mask if port == 'B' else 1)
    assert_close(ga, ga_want.double().cpu().numpy(), torch.float32, 'grad A')
    assert_close(gb, gb_want.double().cpu().numpy(), torch.float32, 'grad B')


@pytest.mark.parametrize('batch', [None, 4])
@pytest.mark.parametrize('compressed', [False, True])
def test_sparse_softmax_operator(batch, compressed, gpu, H=128, W=256):
    shape = (H, W) if batch is None else (batch, H, W)
    x_np, x = randn(shape, 12, scale=3.0)
    g_np, g = randn(shape, 13)
    mask_np = ops.block_mask((H, W), (8, 8), 0.9, seed=14)
    mask = torch.from_numpy(mask_np).to(gpu)
    T = float(np.sqrt(W))
    op = sparta.nn.SparseSoftmax(mask, temperature=T, compressed=compressed)
    cfg = {'_impl': 'sparta', 'BLOCK_SIZE_H_VALUE': 32, 'BLOCK_SIZE_W_VALUE': 32, 'ROW_TILE_VALUE': 4}
    sample = x.to(gpu)
    op.build({'forward:y': dict(cfg), 'backward:x': dict(cfg)}, sample_inputs=[sample])
    idx = op.get_sparse_indexes('y')
    xin = (x.to(gpu) * mask)
    if compressed:
        xin = idx.convert(xin)
    xin.requires_grad_(True)
    y = op(xin)
    y_dense = idx.inverse(y) if compressed else y
    want_y = ops.softmax_forward_reference(x_np, mask_np, T)
    assert_close(y_dense.reshape(shape), want_y, torch.float32, 'softmax op forward')
    gin = g.to(gpu) * mask
    y.backward((idx.convert(gin) if compressed else gin).reshape(y.shape))
    gx = idx.inverse(xin.grad) if compressed else xin.grad
    want_gx = ops.softmax_backward_reference(g_np, y_dense.detach().double().cpu().numpy().reshape(shape), mask_np, T)
    assert_close(gx.reshape(shape), want_gx, torch.float32, 'softmax op backward')


def test_tune_grid_builds_best_config(gpu):
    M, K, N = 256, 128, 128
    x_np, x = randn((M, K), 15)
    w_np, w = randn((N, K), 16)
    mask_np = ops.block_mask((N, K), (16, 16), 0.8, seed=17)
    mask = torch.from_numpy(mask_np).to(gpu)
    lin = dense_linear(K, N, w * torch.from_numpy(mask_np), None, gpu)
    op = sparta.nn.SparseLinear(lin, weight_mask=mask)
    best = sparta.nn.tune(op, sample_inputs=[x.to(gpu)], algo='grid', max_trials=12, tile_configs=False)
    cfg = best['root']['forward:C']
    assert {'_impl', 'BLOCK_SIZE_M_VALUE', 'BLOCK_SIZE_K_VALUE', 'BLOCK_SIZE_N_VALUE'} <= set(cfg)
    want = ops.matmul_reference(x_np[None], w_np[None], None, mode='dsd', transpose_A=False, transpose_B=True,
                                mask=mask_np, dtype=np.float64)[0]
    assert_close(op(x.to(gpu)), want, torch.float32, 'tuned op')
    # the same config builds a fresh operator through sparta.nn.build
    op2 = sparta.nn.SparseLinear(dense_linear(K, N, w * torch.from_numpy(mask_np), None, gpu), weight_mask=mask)
    sparta.nn.build(op2, [x.to(gpu)], best)
    assert_close(op2(x.to(gpu)), want, torch.float32, 'built op')


def _tuner_log():
    """Collects the tuner's trial lines ('... => <latency> ms')."""
    import logging
    from sparta_amd.nn import module_tuner
    lines = []

    class Collect(logging.Handler):
        def emit(self, record):
            lines.append(record.getMessage())

    handler = Collect()
    module_tuner._logger.addHandler(handler)
    return lines, lambda: module_tuner._logger.removeHandler(handler)


@pytest.mark.parametrize('tile_configs', [True, 'refine'])
def test_tune_searches_the_tile_configurations(tile_configs, gpu):
    """tune(tile_configs=...) really enumerates the library's tile table, on device time:
    every configuration id shows up as a trial, configurations the library refuses for this
    layout count as infinitely slow trials, the winner is written as TILE_CFG into a config
    that build() accepts, and the tuned operator still matches the oracle (forward and the
    gradient of the input)."""
    from sparta_amd import _lib
    M, K, N = 512, 256, 256
    x_np, x = randn((M, K), 15, torch.float16)
    w_np, w = randn((N, K), 16, torch.float16)
    g_np, g = randn((M, N), 18, torch.float16)
    mask_np = ops.block_mask((N, K), (32, 32), 0.7, seed=17)
    mask = torch.from_numpy(mask_np).to(gpu)
    lin = dense_linear(K, N, w * torch.from_numpy(mask_np), None, gpu, torch.float16)
    op = sparta.nn.SparseLinear(lin, weight_mask=mask)
    lines, stop = _tuner_log()
    try:
        best = sparta.nn.tune(op, sample_inputs=[x.to(gpu)], sample_grads=[g.to(gpu)], algo='grid', max_trials=10 ** 6,
                              backward_weight=1.0, tile_configs=tile_configs, verbose=True)
    finally:
        stop()
    config = best['root']
    assert set(config) == {'forward:C', 'backward:A', 'backward:B'}
    trials = [l for l in lines if '=> ' in l]
    failed = [l for l in trials if '=> inf' in l]
    n_spmm, n_dds = (len(_lib.tile_configs(op_id)) for op_id in (_lib.OP_SPMM, _lib.OP_DDS))
    # the reference's space per kernel: 3 x 3 upper points (the two tile dims are shared) x one
    # free block size, + the single point of the 'openai' slot (test/unit/test_tuners.py:58-61)
    if tile_configs is True:
        # joint search: every lower space is multiplied by the kernel's tile table
        assert len(trials) == (9 * 3 + 1) * (n_spmm + n_spmm + n_dds)
    else:
        # the reference's space first, then the tile table once per kernel
        assert len(trials) == (9 * 3 + 1) * 3 + (n_spmm + n_spmm + n_dds)
    # the thin-operand kernel (tile config 9) takes 64 / 128 rows of m only: refused for M = 512
    assert failed and len(failed) < len(trials)
    chosen = {name: cfg.get('TILE_CFG', 0) for name, cfg in config.items()}
    assert all(0 <= c < n_spmm for c in chosen.values())
    # reference configs carry no TILE_CFG: building one resets the kernels to the library's choice
    want = ops.matmul_reference(x_np[None], w_np[None], None, mode='dsd', transpose_A=False, transpose_B=True,
                                mask=mask_np, dtype=np.float64)[0]
    for name, cfg in config.items():
        kernel = op._sparse_ctx._kernels[name].active_kernel()
        assert int(kernel.get_parameter('TILE_CFG') or 0) == chosen[name]
    xg = x.to(gpu).requires_grad_(True)
    y = op(xg)
    assert_close(y, want, torch.float16, f'tuned op, tile configs {chosen}')
    y.backward(g.to(gpu))
    want_gx = g_np @ (w_np * mask_np)
    assert_close(xg.grad, want_gx, torch.float16, 'tuned op, input gradient', scale=float(np.abs(want_gx).max()))
    op2 = sparta.nn.SparseLinear(dense_linear(K, N, w * torch.from_numpy(mask_np), None, gpu, torch.float16), weight_mask=mask)
    sparta.nn.build(op2, [x.to(gpu)], best)
    assert_close(op2(x.to(gpu)), want, torch.float16, 'built from the tuned config')
    plain = {name: {k: v for k, v in cfg.items() if k != 'TILE_CFG'} for name, cfg in config.items()}
    op2.build(plain, sample_inputs=[x.to(gpu)])
    assert all(int(op2._sparse_ctx._kernels[n].active_kernel().get_parameter('TILE_CFG') or 0) == 0 for n in plain)


def test_tune_tile_configurations_of_softmax_attention_and_moe(gpu):
    """The softmax kernels' TILE_CFG, the fused attention kernel's and the MoE product's tile
    configuration are search entries too; the tuned modules match their references."""
    from sparta_amd import _lib
    H, Nt, Ns, E = 2, 256, 256, 64
    _, q = randn((H, Nt, E), 21, torch.float16)
    _, k = randn((H, Ns, E), 22, torch.float16)
    _, v = randn((H, Ns, E), 23, torch.float16)
    mask_np = ops.block_mask((Nt, Ns), (32, 32), 0.6, seed=24)
    att = sparta.nn.SparseAttention(mask=torch.from_numpy(mask_np).to(gpu))
    lines, stop = _tuner_log()
    try:
        best = sparta.nn.tune(att, sample_inputs=[q.to(gpu), k.to(gpu), v.to(gpu)], algo='rand', max_trials=3,
                              tile_configs='refine', verbose=True)
    finally:
        stop()
    config = best['root']
    assert 'fused/forward' in config and 0 <= config['fused/forward']['TILE_CFG'] < len(_lib.tile_configs(_lib.OP_ATTENTION))
    n_sm = len(_lib.tile_configs(_lib.OP_SOFTMAX))
    assert sum('[Kernel: sm/forward:y] tile config' in l for l in lines) == n_sm
    want = ops.attention_reference(*(t.double().numpy() for t in (q, k, v)), mask_np)
    with torch.no_grad():
        assert_close(att(q.to(gpu), k.to(gpu), v.to(gpu)), want, torch.float16, 'tuned attention (fused)')
        att._fused = False
        assert_close(att(q.to(gpu), k.to(gpu), v.to(gpu)), want, torch.float16, 'tuned attention (three operators)')
    att2 = sparta.nn.SparseAttention(mask=torch.from_numpy(mask_np).to(gpu))
    sparta.nn.build(att2, [q.to(gpu), k.to(gpu), v.to(gpu)], best)
    assert att2._fused_tile_cfg == config['fused/forward']['TILE_CFG']

    class Net(torch.nn.Module):
        def __init__(self, moe):
            super().__init__()
            self.moe = moe

        def forward(self, tokens, ids):
            return self.moe(tokens, ids)

    torch.manual_seed(3)
    experts = [torch.nn.Linear(128, 256, bias=False, device=gpu, dtype=torch.float16) for _ in range(4)]
    tokens = torch.randn((512, 128), device=gpu, dtype=torch.float16)
    ids = torch.randint(0, 4, (512,), device=gpu, dtype=torch.int32)
    net = Net(sparta.nn.DynamicSparseMoE(experts))
    best = sparta.nn.tune(net, sample_inputs=[tokens, ids], tile_configs=True)
    assert set(best) == {'root/moe'} and net.moe.tile_cfg == best['root/moe']['forward']['TILE_CFG']
    want = torch.stack([experts[int(e)](t) for t, e in zip(tokens, ids.cpu())])
    torch.testing.assert_close(net(tokens, ids).float(), want.float(), rtol=1e-2, atol=1e-2)
    net2 = Net(sparta.nn.DynamicSparseMoE(experts))
    sparta.nn.build(net2, [tokens, ids], best)
    assert net2.moe.tile_cfg == net.moe.tile_cfg


def test_tune_inside_a_combined_module(gpu):
    class Net(torch.nn.Module):
        def __init__(self, a, b):
            super().__init__()
            self.fc1, self.act, self.fc2 = a, torch.nn.ReLU(), b

        def forward(self, x):
            return self.fc2(self.act(self.fc1(x)))

    torch.manual_seed(0)
    l1 = torch.nn.Linear(128, 256, device=gpu)
    l2 = torch.nn.Linear(256, 64, device=gpu)
    m1 = sparta.testing.block_mask((256, 128), block=(32, 32), sparsity=0.5, device=gpu)
    m2 = sparta.testing.block_mask((64, 256), block=(32, 32), sparsity=0.5, device=gpu)
    with torch.no_grad():
        l1.weight.mul_(m1)
        l2.weight.mul_(m2)
    x = torch.rand((64, 128), device=gpu)
    want = l2(torch.relu(l1(x))).detach()
    net = Net(sparta.nn.SparseLinear(l1, weight_mask=m1), sparta.nn.SparseLinear(l2, weight_mask=m2))
    best = sparta.nn.tune(net, sample_inputs=[x], algo='rand', max_trials=4)
    assert set(best) == {'root/fc1', 'root/fc2'}
    torch.testing.assert_close(net(x), want, rtol=1e-4, atol=1e-4)


def test_dynamic_mode_never_fetches_nnz(gpu):
    """dynamic=True: index rebuild and matmul are enqueued without reading the live
    block count back to the host; the weight stays one dense parameter."""
    M, K, N = 256, 256, 512
    x_np, x = randn((M, K), 18, torch.float16)
    w_np, w = randn((N, K), 19, torch.float16, scale=0.1)
    op = None
    for seed in range(4):
        mask_np = ops.block_mask((N, K), (32, 64), 0.9, seed=seed)
        mask = torch.from_numpy(mask_np).to(gpu)
        if op is None:
            op = sparta.nn.SparseLinear(dense_linear(K, N, w, None, gpu, torch.float16), weight_mask=mask,
                                        dynamic=True)  # 32x64-granular mask: no masked value inside live blocks
            op.build({'forward:C': {'_impl': 'openai', 'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 64,
                                    'BLOCK_SIZE_N_VALUE': 32}}, sample_inputs=[x.to(gpu)])
        else:
            op.update_mask(weight_mask=mask)
        with torch.no_grad():
            y = op(x.to(gpu))
        idx = op.get_sparse_indexes('B')
        assert idx._block_nnz is None, 'the live block count was synchronised to the host'
        assert op.weight.numel() == N * K and (seed == 0 or op.weight is kept)  # dense, never re-compressed
        kept = op.weight
        want = ops.matmul_reference(x_np[None], w_np[None], None, mode='dsd', transpose_A=False,
                                    transpose_B=True, mask=mask_np, dtype=np.float64)[0]
        assert_close(y, want, torch.float16, f'dynamic seed {seed}')
        assert idx.block_nnz == int(mask_np.reshape(N // 32, 32, K // 64, 64).any(axis=(1, 3)).sum())


def test_build_rejects_kernels_that_disagree_on_a_shared_block_shape(gpu):
    """The kernels of one operator that read the same compressed tensor share its index: a
    configuration whose kernels want different block shapes for that tensor is refused (an
    AssertionError, like any invalid combination), and a kernel of an earlier build that no
    longer fits is switched off instead of running on a stale layout."""
    _, A = randn((2, 128, 64), 71, torch.float16)
    _, B = randn((2, 96, 64), 72, torch.float16)
    mask = torch.from_numpy(ops.block_mask((128, 96), (32, 32), 0.5, seed=73)).to(gpu)
    good = {k: dict(CFG32) for k in ('forward:C', 'backward:A', 'backward:B')}
    bad = {k: dict(v) for k, v in good.items()}
    bad['backward:B']['BLOCK_SIZE_M_VALUE'] = 16     # its tile of the sparse tensor becomes 32 x 16
    op = sparta.nn.SparseBatchMatMul(C_mask=mask, transpose_A=False, transpose_B=True, compressed=True)
    with pytest.raises(AssertionError, match='shares'):
        op.build(bad, sample_inputs=[A.to(gpu), B.to(gpu)])
    op.build(good, sample_inputs=[A.to(gpu), B.to(gpu)])
    want = torch.matmul(A.to(gpu).float(), B.to(gpu).float().transpose(1, 2)) * mask
    got = op.get_sparse_indexes('C').inverse(op(A.to(gpu), B.to(gpu)))
    torch.testing.assert_close(got.float(), want, rtol=1e-2, atol=1e-2)
    # a forward-only rebuild with other blocks leaves the backward kernels of the first build behind
    fwd16 = {'forward:C': {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 16, 'BLOCK_SIZE_K_VALUE': 32, 'BLOCK_SIZE_N_VALUE': 16}}
    op.build(fwd16, sample_inputs=[A.to(gpu), B.to(gpu)])
    got = op.get_sparse_indexes('C').inverse(op(A.to(gpu), B.to(gpu)))
    torch.testing.assert_close(got.float(), want, rtol=1e-2, atol=1e-2)
    Ar = A.to(gpu).requires_grad_(True)
    with pytest.raises(ValueError, match='not compiled'):
        op(Ar, B.to(gpu)).sum().backward()
