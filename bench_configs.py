"""Secondary measurements for the benchmark configurations other than the headline
line of bench.py: `python bench.py --config c1|c2|c3|c4|c5|seqlen|ceilings|all`.  Prints one JSON
object per measurement.  Inputs are synthetic, generated on the CPU with fixed
seeds and copied to the GPU."""
import json
import math

import numpy as np


def _grid_attention(n_blocks=64, seed=2022):
    grid = np.zeros((n_blocks, n_blocks), dtype=np.uint8)
    i, j = np.indices(grid.shape)
    grid[(i - j >= 0) & (i - j <= 4)] = 1
    grid |= (np.random.default_rng(seed).random(grid.shape) < 0.02).astype(np.uint8)
    return grid


_RESULTS = []


def _close(torch, got, want, what, rtol=1e-2, atol=1e-2):
    """Every measurement below is preceded by this comparison with a dense fp32 torch
    computation of the same inputs on the GPU; a mismatch aborts the benchmark."""
    try:
        torch.testing.assert_close(got.float(), want.float(), rtol=rtol, atol=atol)
    except AssertionError as exc:
        raise AssertionError(f'{what}: result differs from the dense computation\n{exc}') from None


def _emit(name, sec, flops=None, bytes_alg=None, extra=None):
    out = {'config': name, 'ms': sec * 1e3}
    if _emit.stats:   # statistics of the graph replays that `sec` (the shortest) was taken from
        out.update(_emit.stats)
        _emit.stats = None
    if flops:
        out['effective_tflops'] = flops / sec / 1e12
        out['mfma_frac_fp16_peak'] = flops / sec / 1e12 / 2500.0
    if bytes_alg:
        out['algorithmic_gbs'] = bytes_alg / sec / 1e9
        out['hbm_frac'] = bytes_alg / sec / 1e9 / 8000.0
    out.update(extra or {})
    _RESULTS.append(out)
    if _emit.verbose:
        print(json.dumps(out), flush=True)


_emit.verbose = True
_emit.stats = None


def run(which, steps, warmup, time_graph, time_eager, attention_tile_cfg=0, brief=False, verbose=True):
    """Runs the named configurations ('all', one name, or a list of names); every timed
    operator is first compared with the dense computation.  `brief` leaves out the
    comparison methods (dense torch, unfused pipelines, training steps); `verbose`
    prints one JSON object per measurement.  Returns the list of measurements."""
    import torch
    import sparta_amd as sparta
    from oracle import ops
    from sparta_amd.specializer.kernels import SparTASparseMatMulKernel
    from sparta_amd.tesa import get_bcs_function

    dev = torch.device('cuda:0')
    todo = ['c1', 'c2', 'c3', 'c4', 'c5', 'seqlen'] if which == 'all' else ([which] if isinstance(which, str) else list(which))
    steps = min(steps, 100)
    del _RESULTS[:]
    _emit.verbose = verbose

    def timed(fn):
        # shortest replay out of at least three and at least 50 ms of them: the first ones after
        # the correctness checks run at ramping clocks
        try:
            sec = time_graph(torch, fn, steps, warmup, 3, 0.05) / steps
            last = getattr(time_graph, 'last', None)
            if last:
                _emit.stats = {'ms_mean': last['mean_s'] / steps * 1e3, 'steps_per_replay': steps,
                               'replays': last['replays']}
            return sec
        except Exception:
            _emit.stats = None
            return min(time_eager(torch, fn, steps, warmup) for _ in range(3)) / steps

    cfg32 = {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 32, 'BLOCK_SIZE_N_VALUE': 32}
    with torch.no_grad():
        if 'ceilings' in todo:
            # What plain streaming kernels (the library's probe and torch's own) reach on this machine, for reading the
            # HBM fractions of the memory-bound kernels: a read-only reduction, a write-only
            # fill and a copy, each over 1 GiB (four times the last-level cache).
            n = 1 << 28
            src = torch.empty(n, dtype=torch.float32, device=dev).normal_()
            dst = torch.empty_like(src)
            from sparta_amd import _lib
            lib = _lib.load()
            def probe(mode):
                return lambda: _lib.check(lib.spx_stream_probe(mode, _lib.dev_ptr(src), _lib.dev_ptr(dst), 4 * n,
                                                               _lib.current_stream(dev)), 'spx_stream_probe')
            for name, fn, nbytes in (('ceiling: read-only pass over 1 GiB (16-byte non-temporal loads)', probe(0), 4 * n),
                                     ('ceiling: read-only torch.sum over 1 GiB', lambda: torch.sum(src), 4 * n),
                                     ('ceiling: write-only fill of 1 GiB (torch)', lambda: dst.fill_(1.0), 4 * n),
                                     ('ceiling: copy of 1 GiB (16-byte non-temporal loads and stores)', probe(1), 8 * n),
                                     ('ceiling: copy of 1 GiB (torch)', lambda: dst.copy_(src), 8 * n)):
                _emit(name, timed(fn), bytes_alg=nbytes)
            del src, dst
        if 'c1' in todo:
            g = torch.Generator().manual_seed(2022)
            x = torch.rand((1024, 1024), generator=g).to(dev)
            w = torch.rand((1024, 1024), generator=g)
            b = torch.rand((1024,), generator=g)
            mask_np = ops.block_mask((1024, 1024), (8, 8), 0.9, seed=2022)
            lin = torch.nn.Linear(1024, 1024, device=dev)
            lin.weight.copy_((w * torch.from_numpy(mask_np)).to(dev))
            lin.bias.copy_(b.to(dev))
            want = torch.nn.functional.linear(x, lin.weight, lin.bias)
            for blk in ((16,) if brief else (16, 32)):
                op = sparta.nn.SparseLinear(lin, weight_mask=torch.from_numpy(mask_np).to(dev))
                cfg = dict(cfg32, BLOCK_SIZE_K_VALUE=blk, BLOCK_SIZE_N_VALUE=blk)
                op.build({'forward:C': cfg}, sample_inputs=[x])
                nnz = op.get_sparse_indexes('B').block_nnz
                _close(torch, op(x), want, f'c1 {blk}x{blk}', rtol=1e-4, atol=1e-4)
                sec = timed(lambda: op(x))
                _emit(f'c1 SparseLinear fp32 1024^3 8x8@90%, {blk}x{blk} tiles', sec, flops=2.0 * 1024 * nnz * blk * blk,
                      extra={'nnz_blocks': nnz, 'useful_gflop_8x8': 0.215})
            if not brief:
                sec = timed(lambda: lin(x))
                _emit('c1 dense torch Linear fp32', sec, flops=2.0 * 1024 ** 3)

        if 'c2' in todo:
            M = K = N = 4096
            g = torch.Generator().manual_seed(2022)
            A = torch.randn((1, M, K), generator=g).half().to(dev)
            B = torch.randn((1, N, K), generator=g).half().to(dev)
            mask = torch.from_numpy(ops.block_mask((4096, 4096), (32, 32), 0.95, seed=2022)).to(dev)
            maskf = mask.float()
            for mode in ('sdd', 'dsd', 'dds'):
                k = SparTASparseMatMulKernel(mode=mode, biased=False, transpose_A=False, transpose_B=True, compressed=True)
                port = {'sdd': 'A', 'dsd': 'B', 'dds': 'C'}[mode]
                k.ports[port].set_mask(mask)
                k.set_shape(1, M, K, N)
                k.compile(dict(cfg32))
                idx = k.ports[port].indexes
                args = {'sdd': (idx.convert(A), B), 'dsd': (A, idx.convert(B)), 'dds': (A, B)}[mode]
                nnz = idx.block_nnz
                if mode == 'sdd':
                    want = torch.matmul(A[0].float() * maskf, B[0].float().t())
                elif mode == 'dsd':
                    want = torch.matmul(A[0].float(), (B[0].float() * maskf).t())
                else:
                    want = idx.convert(torch.matmul(A[0].float(), B[0].float().t()))
                _close(torch, k(*args).reshape(want.shape), want, f'c2 {mode}')
                del want
                sec = timed(lambda: k(*args))
                _emit(f'c2 {mode} 4096^3 fp16 32x32@95%', sec, flops=nnz * 2.0 * 4096 * 1024,
                      bytes_alg=2 * 4096 * 4096 * 2 + nnz * 2048, extra={'nnz_blocks': nnz})
            if not brief:
                # the same product with the weight stored [K, N] (transpose_B = False)
                k = SparTASparseMatMulKernel(mode='dsd', biased=False, transpose_A=False, transpose_B=False, compressed=True)
                mask_kn = mask.t().contiguous()
                k.ports['B'].set_mask(mask_kn)
                k.set_shape(1, M, K, N)
                k.compile(dict(cfg32))
                idx = k.ports['B'].indexes
                B_kn = B[0].t().contiguous()[None]
                args = (A, idx.convert(B_kn))
                want = torch.matmul(A[0].float(), B_kn[0].float() * mask_kn.float())
                _close(torch, k(*args).reshape(want.shape), want, 'c2 dsd [K, N]')
                del want
                sec = timed(lambda: k(*args))
                _emit('c2 dsd 4096^3 fp16 32x32@95%, weight stored [K, N]', sec, flops=idx.block_nnz * 2.0 * 4096 * 1024,
                      bytes_alg=2 * 4096 * 4096 * 2 + idx.block_nnz * 2048, extra={'nnz_blocks': idx.block_nnz})
                sec = timed(lambda: torch.matmul(A[0], B[0].t()))
                _emit('c2 dense torch.matmul fp16 4096^3', sec, flops=2.0 * 4096 ** 3)
            from oracle import bcs
            mask_np = mask.cpu().numpy()
            for both in (False, True):
                fn = get_bcs_function(32, 32, True, both)
                built = fn.build_indexes(mask)
                row_ptr, bcsr, _ = bcs.build_bcsr(mask_np, 32, 32)
                assert np.array_equal(built.row_ptr.cpu().numpy(), row_ptr), 'c2 index build: row_ptr differs from the oracle'
                assert np.array_equal(built.BCSR_idx.cpu().numpy(), bcsr), 'c2 index build: BCSR_idx differs from the oracle'
                sec = timed(lambda: fn.build_indexes(mask))
                _emit(f"c2 index build 4096x4096 mask ({'BCSR+BCSC' if both else 'BCSR'})", sec, bytes_alg=4096 * 4096)

        if 'c3' in todo:
            BH, N, E, blk = 96, 4096, 64, 64
            grid = _grid_attention()
            mask = torch.from_numpy(np.kron(grid, np.ones((blk, blk), dtype=np.uint8))).to(dev)
            g = torch.Generator().manual_seed(2022)
            q, k_, v = (torch.randn((BH, N, E), generator=g).half().to(dev) for _ in range(3))
            att = sparta.nn.SparseAttention(mask=mask, fused_tile_cfg=attention_tile_cfg)
            mm = {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 64, 'BLOCK_SIZE_K_VALUE': 32, 'BLOCK_SIZE_N_VALUE': 64}
            att.build({'qk/forward:C': dict(mm),
                       'sm/forward:y': {'_impl': 'sparta', 'BLOCK_SIZE_H_VALUE': 64, 'BLOCK_SIZE_W_VALUE': 64, 'ROW_TILE_VALUE': 4},
                       'out/forward:C': {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 64, 'BLOCK_SIZE_K_VALUE': 64, 'BLOCK_SIZE_N_VALUE': 32}},
                      sample_inputs=[q, k_, v])
            nnz = att._sparse_port.indexes.block_nnz
            flops = 2 * nnz * 2.0 * blk * blk * E * BH
            sample = [0, 42, 95]
            scores = torch.matmul(q[sample].float(), k_[sample].float().transpose(1, 2)) / math.sqrt(E)
            scores.masked_fill_(mask == 0, float('-inf'))
            want = torch.matmul(torch.softmax(scores, -1), v[sample].float())
            del scores
            _close(torch, att(q, k_, v)[sample], want, 'c3 fused attention (heads 0, 42, 95)')
            sec = timed(lambda: att(q, k_, v))
            _emit('c3 fused sparse attention 96x4096x64 fp16, 64x64 blocks', sec, flops=flops,
                  bytes_alg=4 * BH * N * E * 2, extra={'nnz_blocks': nnz, 'tile_cfg': attention_tile_cfg})
            # the masked block softmax on the compressed scores of the same problem (read + write of
            # the live entries: the HBM-bound kernel of the three-operator pipeline)
            scores_c = att._matmul_qk.forward(q, k_)
            probs_c = att._softmax.forward(scores_c)
            idx = att._sparse_port.indexes
            dense_scores = torch.matmul(q[sample].float(), k_[sample].float().transpose(1, 2)) / math.sqrt(E)
            dense_scores.masked_fill_(mask == 0, float('-inf'))
            _close(torch, idx.inverse(probs_c[sample]), torch.softmax(dense_scores, -1), 'c3 softmax (heads 0, 42, 95)')
            del dense_scores
            sec = timed(lambda: att._softmax.forward(scores_c))
            _emit('c3 masked block softmax on the compressed scores, 96 x 391 blocks of 64x64 fp16', sec,
                  bytes_alg=2 * scores_c.numel() * 2, extra={'nnz_blocks': nnz})
            del scores_c, probs_c
        if 'c3' in todo and not brief:
            att._fused = False
            _close(torch, att(q, k_, v)[sample], want, 'c3 three-operator pipeline (heads 0, 42, 95)')
            sec = timed(lambda: att(q, k_, v))
            _emit('c3 three-operator pipeline (dds, softmax, sdd)', sec, flops=flops)
            qq, kk, vv = (t.view(8, 12, N, E) for t in (q, k_, v))
            sec = timed(lambda: torch.nn.functional.scaled_dot_product_attention(qq, kk, vv))
            _emit('c3 dense torch SDPA (no mask)', sec, flops=4.0 * BH * N * N * E)
            # one training step (forward + backward, gradients of q, k, v) on the same problem
            with torch.enable_grad():
                sq = {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 64, 'BLOCK_SIZE_K_VALUE': 64, 'BLOCK_SIZE_N_VALUE': 64}
                sm = {'_impl': 'sparta', 'BLOCK_SIZE_H_VALUE': 64, 'BLOCK_SIZE_W_VALUE': 64, 'ROW_TILE_VALUE': 4}
                leaves = [t.clone().requires_grad_(True) for t in (q, k_, v)]
                grad = torch.randn((BH, N, E), generator=g).half().to(dev)
                att_t = sparta.nn.SparseAttention(mask=mask)
                att_t.build({f'{part}/{pas}': dict(sq) for part in ('qk', 'out') for pas in ('forward:C', 'backward:A', 'backward:B')}
                            | {'sm/forward:y': dict(sm), 'sm/backward:x': dict(sm)}, sample_inputs=leaves)

                def step(fn):
                    for t in leaves:
                        t.grad = None
                    fn(*leaves).backward(grad)

                n_step = min(steps, 20)
                for fused, recompute, name in (
                        (True, True, 'c3 training step, no stored probabilities (forward with row statistics, recomputing row-side and column-side backward kernels)'),
                        (True, False, 'c3 training step, stored probabilities (fused forward, row-side and column-side backward kernels)'),
                        (False, False, 'c3 training step, three operators forward and six kernels backward')):
                    att_t._fused = fused
                    att_t._recompute = recompute
                    sec = min(time_eager(torch, lambda: step(att_t), n_step, 3) for _ in range(3)) / n_step
                    _emit(name, sec, flops=3 * flops)
                dense = lambda a, b, c: torch.nn.functional.scaled_dot_product_attention(
                    a.view(8, 12, N, E), b.view(8, 12, N, E), c.view(8, 12, N, E)).view(BH, N, E)
                sec = time_eager(torch, lambda: step(dense), n_step, 3) / n_step
                _emit('c3 training step, dense torch SDPA (no mask)', sec, flops=3 * 4.0 * BH * N * N * E)

        if 'c4' in todo:
            T, D, F = 8192, 768, 3072
            g = torch.Generator().manual_seed(2022)
            x = torch.randn((T, D), generator=g).half().to(dev)
            l1 = torch.nn.Linear(D, F, bias=False, device=dev, dtype=torch.float16)
            l2 = torch.nn.Linear(F, D, bias=False, device=dev, dtype=torch.float16)
            l1.weight.copy_((0.02 * torch.randn((F, D), generator=g)).half().to(dev))
            l2.weight.copy_((0.02 * torch.randn((D, F), generator=g)).half().to(dev))

            def topk_mask(shape, seed):
                rows, cols = shape[0] // 32, shape[1] // 64
                score = torch.randn((rows, cols), generator=torch.Generator().manual_seed(seed)).abs()
                keep = math.ceil(0.1 * rows * cols)
                thr = score.flatten().topk(keep).values[-1]
                grid = (score >= thr).to(torch.uint8)
                return grid.repeat_interleave(32, 0).repeat_interleave(64, 1).contiguous().to(dev)

            masks1 = [topk_mask((F, D), s) for s in range(4)]
            masks2 = [topk_mask((D, F), 100 + s) for s in range(4)]
            cfg = {'forward:C': {'_impl': 'openai', 'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 64, 'BLOCK_SIZE_N_VALUE': 32}}
            def dense_ffn(m1, m2):
                h = torch.relu(torch.matmul(x.float(), (l1.weight.float() * m1.float()).t())).half()
                return torch.matmul(h.float(), (l2.weight.float() * m2.float()).t())

            for dynamic in ((True,) if brief else (True, False)):
                # the activation between the layers runs in the first layer's epilogue
                op1 = sparta.nn.SparseLinear(l1, weight_mask=masks1[0], dynamic=dynamic, activation='relu')
                op2 = sparta.nn.SparseLinear(l2, weight_mask=masks2[0], dynamic=dynamic)
                op1.build(cfg, sample_inputs=[x])
                op2.build(cfg, sample_inputs=[op1(x)])
                m1 = masks1[1].clone()
                m2 = masks2[1].clone()

                def step():
                    # the two rebuilds are independent: one library call, one pair of launches
                    sparta.nn.update_masks([(op1, {'weight_mask': m1}), (op2, {'weight_mask': m2})])
                    return op2(op1(x))

                _close(torch, step(), dense_ffn(m1, m2), f'c4 dynamic={dynamic}')
                if dynamic:
                    sec = timed(step)  # no host sync inside: capturable
                    # a new mask in the same buffers: the next call rebuilds both indexes from it
                    m1.copy_(masks1[2])
                    m2.copy_(masks2[2])
                    _close(torch, step(), dense_ffn(masks1[2], masks2[2]), 'c4 after a mask update')
                    tag = 'hip graph replay'
                else:
                    sec = time_eager(torch, step, steps, warmup) / steps
                    tag = 'eager (one host sync per rebuild, as in the reference)'
                _emit(f'c4 dynamic-mask FFN 8192x768->3072->768 fp16, rebuild timed, dynamic={dynamic}', sec,
                      flops=2 * 2.0 * T * 116 * 32 * 64, extra={'timing': tag})
            if not brief:
                fwd_only = timed(lambda: op2(op1(x)))
                _emit('c4 same FFN, masks fixed (no rebuild)', fwd_only, flops=2 * 2.0 * T * 116 * 32 * 64)
                op1p = sparta.nn.SparseLinear(l1, weight_mask=m1, dynamic=True)
                op2p = sparta.nn.SparseLinear(l2, weight_mask=m2, dynamic=True)
                op1p.build(cfg, sample_inputs=[x])
                op2p.build(cfg, sample_inputs=[torch.relu(op1p(x))])

                def step_unfused():
                    op1p.update_mask(weight_mask=m1)
                    op2p.update_mask(weight_mask=m2)
                    return op2p(torch.relu(op1p(x)))

                _close(torch, step_unfused(), dense_ffn(m1, m2), 'c4 separate activation kernel')
                _emit('c4 dynamic FFN with the activation as a separate torch kernel (as the reference would run it)',
                      timed(step_unfused), flops=2 * 2.0 * T * 116 * 32 * 64)
                sec = timed(lambda: l2(torch.relu(l1(x))))
                _emit('c4 dense torch FFN fp16', sec, flops=2 * 2.0 * T * D * F)

        if 'c5' in todo:
            n_tok, n_exp, K, N = 16384, 8, 1024, 4096
            g = torch.Generator().manual_seed(2022)
            mods = []
            for _ in range(n_exp):
                lin = torch.nn.Linear(K, N, bias=False, dtype=torch.float16, device=dev)
                lin.weight.copy_((0.02 * torch.randn((N, K), generator=g)).half().to(dev))
                mods.append(lin)
            moe = sparta.nn.DynamicSparseMoE(mods)
            p = np.arange(1, n_exp + 1, dtype=np.float64) ** -1.2
            ids = torch.from_numpy(np.random.default_rng(2022).choice(n_exp, size=n_tok, p=p / p.sum()).astype(np.int32)).to(dev)
            x = torch.randn((n_tok, K), generator=g).half().to(dev)
            got = moe(x, ids)
            want = torch.empty((n_tok, N), dtype=torch.float32, device=dev)
            for e in range(n_exp):
                rows = (ids == e).nonzero().flatten()
                want[rows] = torch.matmul(x[rows].float(), mods[e].weight.float().t())
            _close(torch, got, want, 'c5 MoE forward')
            del want, got
            sec = timed(lambda: moe(x, ids))
            _emit('c5 MoE forward 16384 tok, 1024->4096, 8 experts Zipf(1.2), index rebuild included', sec,
                  flops=2.0 * n_tok * K * N, bytes_alg=(n_tok * K + n_exp * K * N + n_tok * N) * 2,
                  extra={'expert_counts': moe.expert_count.cpu().tolist()})
            if not brief:
                w0 = mods[0].weight
                sec = timed(lambda: torch.matmul(x, w0.t()))
                _emit('c5 dense torch.matmul with the same FLOPs (16384x1024x4096)', sec, flops=2.0 * n_tok * K * N)

        if 'seqlen' in todo:
            # SeqlenDynamicSparseAttention: the reference test's shape (fp32) and a larger fp16 one;
            # lengths uniform in [1, N); dense SDPA over the padded batch for comparison
            for (B, H, N, E), dtype in (((12, 20, 256, 64), torch.float32), ((32, 12, 1024, 64), torch.float16)):
                g = torch.Generator().manual_seed(2022)
                q, k_, v = (torch.rand((B, H, N, E), generator=g).to(dtype).to(dev) for _ in range(3))
                lens = np.random.default_rng(2022).integers(1, N, size=B).astype(np.int32)
                seqlens = torch.from_numpy(lens).to(dev)
                att = sparta.nn.SeqlenDynamicSparseAttention(global_mode=False)
                flops = float(sum(4.0 * int(L) * int(L) * E * H for L in lens))
                got = att(q, k_, v, seqlens)
                for b in (0, B // 2, B - 1):
                    L = int(lens[b])
                    p = torch.softmax(torch.matmul(q[b, :, :L].float(), k_[b, :, :L].float().transpose(1, 2)), -1)
                    tol = 1e-4 if dtype == torch.float32 else 1e-2
                    _close(torch, got[b, :, :L], torch.matmul(p, v[b, :, :L].float()), f'seqlen attention b={b}', tol, tol)
                    assert float(got[b, :, L:].abs().max()) == 0.0, 'seqlen attention: rows past the length are not zero'
                sec = timed(lambda: att(q, k_, v, seqlens))
                name = str(dtype).replace('torch.', '')
                _emit(f'seqlen attention {B}x{H}x{N}x{E} {name}, lengths uniform in [1, {N})', sec, flops=flops,
                      bytes_alg=float(sum(4 * int(L) * E * H for L in lens)) * q.element_size())
                if not brief:
                    sec = timed(lambda: torch.nn.functional.scaled_dot_product_attention(q, k_, v, scale=1.0))
                    _emit(f'seqlen shape, dense torch SDPA over the padded batch ({name})', sec, flops=4.0 * B * H * N * N * E)
    return list(_RESULTS)

