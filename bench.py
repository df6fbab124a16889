#!/usr/bin/env python
"""Headline benchmark: block-sparse linear 4096x4096x4096 fp16, 32x32 blocks, 95% sparse.

One step = one forward pass of `SparseLinear(weight_mask=...)` (the 'dsd' kernel,
weight stored [N, K] and BCSR-compressed) over one resident input batch.  The K
timed steps are captured once in a HIP graph and replayed, so the measurement is
the device time of the kernels and not the Python launch path; the eager
per-call latency is reported next to it.

Prints ONE JSON line: effective TFLOP/s counted on the non-zero blocks (`value`),
ms per step, the dense torch.matmul time on the same GPU, the HBM roofline of
the matmul kernel and a CPU baseline (the numpy oracle's masked-dense product
timed on the host cores).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

M = K = N = 4096
BLOCK = (32, 32)
SPARSITY = 0.95
SEED = 2022
SETTLE_S = 0.1   # untimed replays before the timed region (seconds of device time)
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0  # dense fp16


def make_inputs(torch, device):
    g = torch.Generator().manual_seed(SEED)
    x = torch.randn((M, K), generator=g).half()
    w = torch.randn((N, K), generator=g).half()
    from oracle import ops
    mask = ops.block_mask((N, K), BLOCK, SPARSITY, seed=SEED)
    return x, w, mask


def time_graph(torch, fn, steps, warmup, repeats=1, min_total=0.0, settle=0.0):
    """Device time of `steps` calls of fn(), replayed from one captured graph and
    bracketed by events on the replay stream.  Returns seconds for all steps (the
    shortest of the timed replays: at least `repeats` of them, and as many more as
    it takes to spend `min_total` seconds of device time, so that a short graph is
    also timed at settled clocks).  `settle` > 0 replays the graph untimed for that many
    seconds of device time first: the clocks of an idle GPU ramp for tens of milliseconds,
    longer than a short timed region lasts.  `time_graph.last` keeps the shortest and the
    mean replay and their number."""
    for _ in range(max(warmup, 1)):
        fn()
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        fn()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(steps):
                fn()
        graph.replay()  # untimed replay: page in the graph
        stream.synchronize()
        spent, rolls = 0.0, 0
        while spent < settle and rolls < 100000:
            begin = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            begin.record(stream)
            for _ in range(8):
                graph.replay()
            end.record(stream)
            stream.synchronize()
            spent += begin.elapsed_time(end) / 1e3
            rolls += 8
        best, total, done = None, 0.0, 0
        while done < max(repeats, 1) or (total < min_total and done < 1000):
            begin = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            begin.record(stream)
            graph.replay()
            end.record(stream)
            stream.synchronize()
            took = begin.elapsed_time(end) / 1e3
            best = took if best is None else min(best, took)
            total += took
            done += 1
    time_graph.last = {'steps': steps, 'replays': done, 'min_s': best, 'mean_s': total / done}
    return best


time_graph.last = None


def time_eager(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    begin = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    begin.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return begin.elapsed_time(end) / 1e3


def cpu_baseline(x, w, mask, nnz):
    """The oracle's masked-dense product (fp32 on the fp16-rounded inputs) on the
    host cores; a bounded number of repetitions of the full-size problem."""
    from oracle import ops
    a = x.float().numpy()[None]
    b = w.float().numpy()[None]
    cores = int(os.environ.get('OMP_NUM_THREADS', os.cpu_count() or 1))
    ops.matmul_reference(a, b, None, mode='dsd', transpose_A=False, transpose_B=True, mask=mask)  # warm-up
    reps, spent = 0, 0.0
    while reps < 3 or (spent < 10.0 and reps < 20):
        t0 = time.perf_counter()
        ops.matmul_reference(a, b, None, mode='dsd', transpose_A=False, transpose_B=True, mask=mask)
        spent += time.perf_counter() - t0
        reps += 1
    per_call = spent / reps
    flops_nz = nnz * 2.0 * M * BLOCK[0] * BLOCK[1]
    return {
        'value': flops_nz / per_call / 1e12,
        'unit': 'TFLOP/s effective on non-zero blocks',
        'ms_per_step': per_call * 1e3,
        'cores': cores,
        'kind': 'port',
        'sample': f'{reps} repetitions of the full 4096^3 masked-dense fp32 product (numpy/BLAS, {cores} threads)',
    }


def measured_traffic_bytes():
    """HBM bytes per launch of the matmul kernel from the committed rocprofv3 --pmc
    summary (FETCH_SIZE + WRITE_SIZE, scaled by a copy kernel of known size), or
    None if that summary is absent."""
    path = os.path.join(ROOT, 'profiles', 'spmm_panel_c2_traffic.json')
    try:
        with open(path) as f:
            return json.load(f)['traffic_bytes_per_launch']
    except (OSError, KeyError, ValueError):
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    # a step takes under 30 us: 2000 + 2000 steps are 0.1 s of device time, enough for the clocks to
    # settle (200 steps after 20 of warm-up measured 6 % slower than the steady state)
    ap.add_argument('--steps', type=int, default=2000)
    ap.add_argument('--warmup', type=int, default=2000)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--calibrate-copy', action='store_true',
                    help='also run one plain 256 MiB device copy, so that a rocprofv3 --pmc run of this '
                         'command shows what FETCH_SIZE / WRITE_SIZE read for a kernel of known traffic')
    ap.add_argument('--config', default='headline',
                    help="'headline' (default, the one JSON line the harness reads) or one of c1..c5 / seqlen / all: "
                         "secondary measurements of the other benchmark configurations; 'ceilings': what plain "
                         "read-only, write-only and copy kernels reach on this machine")
    ap.add_argument('--no-secondary', action='store_true',
                    help="leave out the 'secondary' object (the other benchmark configurations, each checked "
                         'against the dense computation before it is timed) and the cold-operand variant')
    ap.add_argument('--attention-tile-cfg', type=int, default=0,
                    help='tile configuration of the fused attention kernel in --config c3 (0 = the library\'s choice)')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).', file=sys.stderr)
        sys.exit(2)
    if args.config != 'headline':
        import bench_configs
        bench_configs.run(args.config, args.steps, args.warmup, time_graph, time_eager, args.attention_tile_cfg)
        return

    import torch
    import sparta_amd as sparta

    if not torch.cuda.is_available():
        print('bench.py needs a GPU', file=sys.stderr)
        sys.exit(2)
    device = torch.device('cuda:0')
    x_cpu, w_cpu, mask_np = make_inputs(torch, device)
    x = x_cpu.to(device)
    mask = torch.from_numpy(mask_np).to(device)

    dense = torch.nn.Linear(K, N, bias=False, device=device, dtype=torch.float16)
    with torch.no_grad():
        dense.weight.copy_(w_cpu.to(device) * mask.half())
    op = sparta.nn.SparseLinear(dense, weight_mask=mask)
    config = {'forward:C': {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 32, 'BLOCK_SIZE_K_VALUE': 32,
                            'BLOCK_SIZE_N_VALUE': 32}}
    op.build(config, sample_inputs=[x])
    nnz = op.get_sparse_indexes('B').block_nnz

    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=device)
        dst = torch.empty_like(src)
        torch.mul(src, 1.0, out=dst)  # one elementwise kernel: 256 MiB read + 256 MiB written
        torch.cuda.synchronize()
        del src, dst

    with torch.no_grad():
        y = op(x)
        ref = torch.matmul(x.float(), (dense.weight.float()).t())
        torch.testing.assert_close(y.float(), ref, rtol=1e-2, atol=1e-2)

        step = lambda: op(x)
        try:
            total = time_graph(torch, step, args.steps, args.warmup, settle=SETTLE_S)
            timing = (f'hip graph replay of the timed steps, events on the replay stream, after the warm-up steps and '
                      f'{SETTLE_S} s of untimed replays of the same graph (an idle GPU ramps its clocks for tens of ms)')
        except Exception as exc:  # capture unsupported: fall back to the eager loop
            total = time_eager(torch, step, args.steps, args.warmup)
            timing = f'eager loop (graph capture failed: {type(exc).__name__})'
        eager = time_eager(torch, step, args.steps, args.warmup)
        w_dense = dense.weight
        dense_total = time_graph(torch, lambda: torch.matmul(x, w_dense.t()), min(args.steps, 100), 5, settle=SETTLE_S)
        dense_ms = dense_total / min(args.steps, 100) * 1e3

        cold = None
        if not args.no_secondary:
            # cold operands: six input / output pairs (402 MB) in rotation, more than the
            # 256 MB of last-level cache, so every x comes from HBM and every y goes there
            ring = 6
            xs = [x] + [x.clone() for _ in range(ring - 1)]
            ys = [None] * ring
            turn = [0]

            def cold_step():
                i = turn[0] % ring
                turn[0] += 1
                ys[i] = op(xs[i])

            cold_steps = max(ring * 4, (args.steps // ring) * ring)
            try:
                cold = time_graph(torch, cold_step, cold_steps, args.warmup, settle=SETTLE_S) / cold_steps
            except Exception:
                cold = time_eager(torch, cold_step, cold_steps, args.warmup) / cold_steps
            torch.testing.assert_close(ys[ring - 1].float(), torch.matmul(xs[ring - 1].float(), dense.weight.float().t()),
                                       rtol=1e-2, atol=1e-2)
            del xs, ys

    sec = total / args.steps
    flops_nz = nnz * 2.0 * M * BLOCK[0] * BLOCK[1]
    # algorithmic bytes of one launch: dense x in, dense y out, live weight blocks, index
    bytes_alg = M * K * 2 + M * N * 2 + nnz * BLOCK[0] * BLOCK[1] * 2 + (N // BLOCK[0] + 1 + nnz) * 4
    out = {
        'metric': 'block-sparse linear 4096^3 fp16 @95% 32x32 sparsity: effective TFLOP/s on non-zero blocks',
        'value': flops_nz / sec / 1e12,
        'unit': 'TFLOP/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': sec * 1e3,
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f16 (fp32 accumulate)',
        'data': 'synthetic',
        'config': {'workload': 'SparseLinear dsd 4096x4096x4096 fp16, 32x32 blocks, 95% sparse (configs[1])',
                   'M': M, 'K': K, 'N': N, 'block': list(BLOCK), 'sparsity': SPARSITY, 'nnz_blocks': int(nnz),
                   'seed': SEED, 'timing': timing},
        'eager_ms_per_step': eager / args.steps * 1e3,
        'dense_torch_matmul_ms': dense_ms,
        'speedup_vs_dense': dense_ms / (sec * 1e3),
        'mfma_frac_nonzero_work': flops_nz / sec / 1e12 / MFMA_PEAK_TFLOPS,
        'roofline': {
            'bound': 'hbm',
            'achieved': bytes_alg / sec / 1e9,
            'peak': HBM_PEAK_GBS,
            'unit': 'GB/s',
            'frac': bytes_alg / sec / 1e9 / HBM_PEAK_GBS,
            'traffic': measured_traffic_bytes(),
            'kernel': 'sparse-operand matmul (dsd)',
            'algorithmic_bytes': int(bytes_alg),
        },
    }
    if cold is not None:
        out['cold_operands'] = {
            'ms_per_step': cold * 1e3,
            'hbm_frac': bytes_alg / cold / 1e9 / HBM_PEAK_GBS,
            'note': 'same step over six rotating x / y pairs (402 MB, beyond the 256 MB last-level cache)',
        }
    if not args.no_secondary:
        import bench_configs
        try:
            sec_steps = min(args.steps, 50)
            rows = bench_configs.run(['c1', 'c2', 'c3', 'c4', 'c5'], sec_steps, min(args.warmup, 10), time_graph,
                                     time_eager, brief=True, verbose=False)
            out['secondary'] = {
                'note': 'other benchmark configurations; each result was compared with the dense fp32 torch '
                        f'computation of the same inputs before it was timed; a replay is one graph of {sec_steps} '
                        'steps, replayed at least three times and for at least 50 ms: "ms" is the shortest replay '
                        '(the first short replays right after the checks run at ramping clocks), "ms_mean" the '
                        'mean over all "replays" (the statistic of the reference\'s profile())',
                'results': [{k: (round(v, 5) if isinstance(v, float) else v) for k, v in r.items()
                             if k != 'expert_counts'} for r in rows],
            }
        except AssertionError as exc:
            out['secondary'] = {'error': str(exc)[:400]}
    if not args.no_cpu_baseline:
        out['cpu_baseline'] = cpu_baseline(x_cpu, w_cpu, mask_np, int(nnz))
    print(json.dumps(out))


if __name__ == '__main__':
    main()
