#!/usr/bin/env python
"""Sparsity x granularity sweeps of the block-sparse matmul and attention operators
against their dense counterparts, in the shape of the reference's
test/bench/matmul/matmul.py and test/bench/attention/attention.py (same problem
sizes, granularities, sparsities, forward and backward latency, one CSV row per
method and point; the Triton competitors are left out).

    python bench_sweep.py --op matmul                    # packaged configs, fp16
    python bench_sweep.py --op matmul --dtype fp32       # the reference's dtype
    python bench_sweep.py --op attention --quick
    python bench_sweep.py --op matmul --tune 8           # tune every point (8 trials per
                                                         # kernel), write params/<device>.csv
    python bench_sweep.py --op matmul --tune 1000 --algo grid   # the whole search space

Operator configurations come from the tuned-config tables shipped in
sparta_amd/params/<op>/ (`<device name>.csv`, else `default.csv`; the format of the
reference's test/bench/*/params/default.csv).  With --tune the tables are
regenerated on this GPU into --out: block sizes by the tuner's search over the reference's
space, then the gfx950 tile configuration of every kernel with those block sizes kept
(tune(..., tile_configs='refine'); every trial is timed on the device).  Results go to
<out>/sweep_<op>_<dtype>.csv.
"""
import argparse
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

GRANULARITY_LIST = [1, 8, 32]
SPARSITY_LIST = [0, 0.2, 0.4, 0.6, 0.8, 0.9, 0.95, 0.99, 0.995, 0.999, 0.9995, 0.9999]
QUICK_SPARSITY = [0, 0.8, 0.95, 0.999]
MATMUL_SHAPE = (3072, 768, 4096)      # M, K, N   (matmul.py:15)
ATTENTION_SHAPE = (4096, 3072, 768)   # Ns, Nt, E (attention.py:18)

_MM = lambda m, k, n: {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': m, 'BLOCK_SIZE_K_VALUE': k, 'BLOCK_SIZE_N_VALUE': n}
_SM = {'_impl': 'sparta', 'BLOCK_SIZE_H_VALUE': 32, 'BLOCK_SIZE_W_VALUE': 32, 'ROW_TILE_VALUE': 4}
MATMUL_FALLBACK = {'forward:C': _MM(32, 32, 32), 'backward:A': _MM(32, 32, 32), 'backward:B': _MM(32, 32, 32)}
ATTENTION_FALLBACK = {'qk/forward:C': _MM(32, 32, 32), 'qk/backward:A': _MM(32, 32, 32), 'qk/backward:B': _MM(32, 32, 32),
                      'sm/forward:y': dict(_SM), 'sm/backward:x': dict(_SM),
                      'out/forward:C': _MM(32, 32, 32), 'out/backward:A': _MM(32, 32, 32), 'out/backward:B': _MM(32, 32, 32)}


def matmul_data(torch, sparta, M, K, N, granularity, sparsity, dtype, device):
    """matmul.py:56-79: B [N, K] masked, C = A B^T, gradients of a random grad_C."""
    torch.manual_seed(2022)
    A = torch.rand((1, M, K), device=device).to(dtype)
    B = torch.rand((1, N, K), device=device).to(dtype)
    mask = sparta.testing.block_mask((N, K), granularity, sparsity, device=device)
    B = B * mask
    grad_C = torch.rand((1, M, N), device=device).to(dtype)
    C = torch.matmul(A.float(), B.float().transpose(1, 2))
    grad_A = torch.matmul(grad_C.float(), B.float())
    grad_B = torch.matmul(grad_C.float().transpose(1, 2), A.float())
    return dict(A=A, B=B, C=C.to(dtype), grad_C=grad_C, grad_A=grad_A.to(dtype), grad_B=grad_B.to(dtype)), mask


def _granularities(args):
    return [args.granularity] if getattr(args, 'granularity', None) else GRANULARITY_LIST


def _sparsities(args):
    if getattr(args, 'sparsity', None) is not None:
        return [args.sparsity]
    return QUICK_SPARSITY if args.quick else SPARSITY_LIST


def time_fwd_bwd(torch, sparta, func, inputs, grad, targets, warmups, iters, grad_targets=None):
    """Forward latency and (forward + backward) - forward, like profile_matmul (matmul.py:25-53).
    Before anything is timed the output is checked against `targets` and the input
    gradients against `grad_targets` (the reference's bench checks both, matmul.py:30-36);
    a mismatch raises AssertionError."""
    def steady(f, args, warm, n, targets=None):
        # shortest block out of at least three and at least 50 ms of them: the first blocks after
        # the set-up of a point run at ramping clocks
        best = sparta.testing.profile(f, args, target_outputs=targets, num_warmups=warm, num_iters=n)
        spent, blocks = best * n, 1
        while (blocks < 3 or spent < 50.0) and blocks < 100 and best != float('inf'):
            t = sparta.testing.profile(f, args, num_warmups=0, num_iters=n)
            best, spent, blocks = min(best, t), spent + t * n, blocks + 1
        return best

    fwd = steady(func, inputs, warmups, iters, targets[:1] if targets else None)
    leaves = [t.detach().clone().requires_grad_(True) for t in inputs]
    if grad_targets is not None:
        func(*leaves).backward(grad)
        for leaf, want in zip(leaves, grad_targets):
            half = leaf.dtype in (torch.float16, torch.bfloat16)
            tol = 1e-2 if half else 1e-4
            # gradients are sums over up to thousands of products: scale the absolute bound by their size
            scale = max(float(want.float().abs().max()), 1.0)
            torch.testing.assert_close(leaf.grad.float(), want.float(), rtol=tol, atol=tol * scale)

    def both(*args):
        for leaf in leaves:
            leaf.grad = None
        out = func(*leaves)
        out.backward(grad)
        return out

    total = steady(both, [], max(warmups // 4, 2), max(iters // 4, 5))
    return fwd, max(total - fwd, 0.0)


def sweep_matmul(args, torch, sparta, table_dir, device_name):
    from sparta_amd.common import config_table as ct
    M, K, N = MATMUL_SHAPE
    dtype = {'fp16': torch.float16, 'fp32': torch.float32, 'bf16': torch.bfloat16}[args.dtype]
    table = None if args.tune else ct.load_config_table(table_dir, device_name)
    rows, tuned = [], []
    for g in _granularities(args):
        for s in _sparsities(args):
            t0 = time.time()
            data, mask = matmul_data(torch, sparta, M, K, N, (g, g), s, dtype, 'cuda')
            dense = lambda A, B: torch.matmul(A, B.transpose(1, 2))
            lat_dense = time_fwd_bwd(torch, sparta, dense, [data['A'], data['B']], data['grad_C'], None,
                                     args.warmups, args.iters)
            rows.append(('dense', M, K, N, g, s) + lat_dense)
            if int(mask.sum()) == 0:
                rows.append(('sparta_amd', M, K, N, g, s, 0.0, 0.0))
                if args.tune:
                    tuned.append(({'granularity': g, 'sparsity': s}, MATMUL_FALLBACK))
                continue
            op = sparta.nn.SparseBatchMatMul(B_mask=mask, transpose_A=False, transpose_B=True, compressed=True)
            sample = [data['A'], data['B']]
            if args.tune:
                best = sparta.nn.tune(op, sample_inputs=sample, sample_grads=[data['grad_C']], algo=args.algo,
                                      max_trials=args.tune, backward_weight=1.0, tile_configs='refine')
                config = best['root']
                if config is None:
                    config = MATMUL_FALLBACK
                    op.build(config, sample_inputs=sample)
                tuned.append(({'granularity': g, 'sparsity': s}, config))
            else:
                config = ct.lookup_config(table, granularity=g, sparsity=s)
                op.build(config, sample_inputs=sample)
            indexes = op.get_sparse_indexes('B')
            Bc = indexes.convert(data['B'])
            # the gradient of the compressed operand covers the live blocks only
            lat = time_fwd_bwd(torch, sparta, op, [data['A'], Bc], data['grad_C'],
                               [data['C']], args.warmups, args.iters,
                               grad_targets=[data['grad_A'], indexes.convert(data['grad_B'])])
            rows.append(('sparta_amd', M, K, N, g, s) + lat)
            print(f'matmul g={g} s={s}: dense fwd {lat_dense[0]*1e3:.1f} us bwd {lat_dense[1]*1e3:.1f} us | '
                  f'sparse fwd {lat[0]*1e3:.1f} us bwd {lat[1]*1e3:.1f} us  ({time.time()-t0:.1f} s)', flush=True)
    return ['method', 'M', 'K', 'N', 'granularity', 'sparsity', 'forward', 'backward'], rows, tuned


def sweep_attention(args, torch, sparta, table_dir, device_name):
    from sparta_amd.common import config_table as ct
    Ns, Nt, E = ATTENTION_SHAPE
    dtype = {'fp16': torch.float16, 'fp32': torch.float32, 'bf16': torch.bfloat16}[args.dtype]
    table = None if args.tune else ct.load_config_table(table_dir, device_name)
    rows, tuned = [], []
    for g in _granularities(args):
        for s in _sparsities(args):
            t0 = time.time()
            torch.manual_seed(2022)
            q = torch.rand((1, Nt, E), device='cuda').to(dtype)
            k = torch.rand((1, Ns, E), device='cuda').to(dtype)
            v = torch.rand((1, Ns, E), device='cuda').to(dtype)
            grad = torch.rand((1, Nt, E), device='cuda').to(dtype)
            mask = sparta.testing.block_mask((Nt, Ns), (g, g), s, device='cuda')
            want = sparta.testing.sparse_multi_head_attention_reference(q.float(), k.float(), v.float(), mask).to(dtype)

            def dense(q, k, v):
                p = torch.matmul(q, k.transpose(1, 2)) / (E ** 0.5)
                p = torch.softmax(p.masked_fill(mask == 0, float('-inf')), -1).nan_to_num(0.0)
                return torch.matmul(p, v)

            lat_dense = time_fwd_bwd(torch, sparta, dense, [q, k, v], grad, None, args.warmups, args.iters)
            rows.append(('dense', Ns, Nt, E, g, s) + lat_dense)
            # gradient targets from the masked dense computation in fp32
            leaves = [t.float().requires_grad_(True) for t in (q, k, v)]
            dense(*leaves).backward(grad.float())
            grad_targets = [leaf.grad for leaf in leaves]
            if int(mask.sum()) == 0:
                rows.append(('sparta_amd', Ns, Nt, E, g, s, 0.0, 0.0))
                if args.tune:
                    tuned.append(({'granularity': g, 'sparsity': s}, ATTENTION_FALLBACK))
                continue
            op = sparta.nn.SparseAttention(mask=mask)
            if args.tune:
                best = sparta.nn.tune(op, sample_inputs=[q, k, v], sample_grads=[grad], algo=args.algo,
                                      max_trials=args.tune, backward_weight=1.0, tile_configs='refine')
                config = best['root']
                if config is None:  # every random trial hit an invalid combination: use the fallback
                    config = ATTENTION_FALLBACK
                    op.build(config, sample_inputs=[q, k, v])
                tuned.append(({'granularity': g, 'sparsity': s}, config))
            else:
                config = ct.lookup_config(table, granularity=g, sparsity=s)
                op.build(config, sample_inputs=[q, k, v])
            lat = time_fwd_bwd(torch, sparta, op, [q, k, v], grad, [want], args.warmups, args.iters,
                               grad_targets=grad_targets)
            rows.append(('sparta_amd', Ns, Nt, E, g, s) + lat)
            print(f'attention g={g} s={s}: dense fwd {lat_dense[0]*1e3:.1f} us bwd {lat_dense[1]*1e3:.1f} us | '
                  f'sparse fwd {lat[0]*1e3:.1f} us bwd {lat[1]*1e3:.1f} us  ({time.time()-t0:.1f} s)', flush=True)
    return ['method', 'Ns', 'Nt', 'E', 'granularity', 'sparsity', 'forward', 'backward'], rows, tuned


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--op', choices=['matmul', 'attention'], default='matmul')
    ap.add_argument('--dtype', choices=['fp16', 'bf16', 'fp32'], default='fp16')
    ap.add_argument('--quick', action='store_true', help='4 sparsities per granularity instead of 12')
    ap.add_argument('--granularity', type=int, default=None, help='run this mask granularity only')
    ap.add_argument('--sparsity', type=float, default=None, help='run this sparsity only')
    ap.add_argument('--tune', type=int, default=0, help='tune every point with this many trials per kernel')
    ap.add_argument('--algo', choices=['rand', 'grid'], default='rand', help='search algorithm of --tune')
    ap.add_argument('--warmups', type=int, default=20)
    ap.add_argument('--iters', type=int, default=50)
    ap.add_argument('--out', default=os.path.join(ROOT, 'sweep_out'), help='directory for the result CSVs')
    args = ap.parse_args()

    import torch
    import sparta_amd as sparta
    from sparta_amd.common import config_table as ct
    if not torch.cuda.is_available():
        print('bench_sweep.py needs a GPU', file=sys.stderr)
        sys.exit(2)
    device_name = torch.cuda.get_device_name(0)
    table_dir = ct.packaged_table_dir(args.op)
    sweep = sweep_matmul if args.op == 'matmul' else sweep_attention
    header, rows, tuned = sweep(args, torch, sparta, table_dir, device_name)
    os.makedirs(args.out, exist_ok=True)
    path = os.path.join(args.out, f'sweep_{args.op}_{args.dtype}.csv')
    with open(path, 'w') as f:
        f.write(','.join(header) + '\n')
        for row in rows:
            f.write(','.join(str(x) for x in row) + '\n')
    print('wrote', path)
    if tuned:
        tpath = os.path.join(args.out, 'params', args.op, f'{device_name}.csv')
        ct.save_config_table(tpath, ['granularity', 'sparsity'], tuned)
        print('wrote', tpath)


if __name__ == '__main__':
    main()
