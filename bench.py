"""
Benchmark of the north-star path: Inception-v3 at batch 1 under the dp_parallel schedule found by the
dynamic-programming search with on-device stage measurements, on one MI355X.

A step is one forward pass over one synthetic batch (weights and input already resident in HBM).  Prints one
JSON line; see DESIGN.md for the definitions behind `roofline` and `cpu_baseline`.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for path in (ROOT, os.path.join(ROOT, 'inter-operator-scheduler_amd')):
    if path not in sys.path:
        sys.path.insert(0, path)

PEAK_FP32_MATRIX_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def network_roofline_ms(ops, parallel):
    """Sum over ops (or over stages of the slowest group) of max(flops / peak, bytes / bandwidth)."""
    def bound(op):
        return max(op['flops'] / (PEAK_FP32_MATRIX_TFLOPS * 1e12), op['bytes'] / (PEAK_HBM_GBS * 1e9)) * 1e3
    if not parallel:
        return sum(bound(op) for op in ops)
    stages = {}
    for op in ops:
        stages.setdefault(op['stage'], {}).setdefault(op['group'], 0.0)
        stages[op['stage']][op['group']] += bound(op)
    return sum(max(groups.values()) for groups in stages.values())


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument('--gpus', type=int, default=1)
    parser.add_argument('--steps', type=int, default=300)
    parser.add_argument('--warmup', type=int, default=30)
    parser.add_argument('--batch', type=int, default=1)
    parser.add_argument('--executor', default=os.environ.get('IOS_BENCH_EXECUTOR', 'fused_graph'),
                        choices=['streams', 'graph', 'fused', 'fused_graph'])
    parser.add_argument('--search-executor', default='fused', choices=['streams', 'fused'],
                        help='executor under which the schedule search measures candidate stages')
    parser.add_argument('--sweep', action='store_true', help='also time batch 16 and 64 with the same schedule')
    parser.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    args = parser.parse_args()
    if args.gpus != 1:
        print('bench.py: this runtime is a single-GPU path; run with --gpus 1', file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import ios
    from ios.contrib import ios_runtime as rt

    device = rt.device_info()
    batch = args.batch
    graph = ios.models.inception_v3(init_seed=0, init_scheme='he_normal')
    x = np.random.default_rng(1).standard_normal((batch, 3, 299, 299)).astype(np.float32)

    # schedule search with measured stage latencies (not part of the timed steps)
    rt.set_option('autotune', 1)        # measure kernel configurations on first sight of a shape
    rt.set_option('executor', args.search_executor)
    t0 = time.time()
    optimized = ios.optimize(graph, batch_size=batch, opt_type='dp_parallel', compute_weight=True,
                             warmup=2, number=6, repeat=3)
    search_s = time.time() - t0
    graph.sequential_schedule()

    rt.set_option('executor', args.executor)

    def timed_latency(g, b, xin, steps, warmup):
        with rt.Session(g, b) as session:
            session.load_weights()
            session.set_input(xin)
            for _ in range(warmup):
                session.run()
            t = time.perf_counter()
            for _ in range(steps):
                session.run()
            wall = (time.perf_counter() - t) / steps * 1e3
            events = session.measure(warmup=2, number=6, repeat=6)
            out = session.output()
            return wall, float(np.mean(events)), float(np.min(events)), float(np.std(events)), out

    seq_wall, seq_ev, seq_min, seq_std, seq_out = timed_latency(graph, batch, x, args.steps, args.warmup)
    opt_wall, opt_ev, opt_min, opt_std, opt_out = timed_latency(optimized, batch, x, args.steps, args.warmup)
    schedule_diff = float(np.abs(seq_out - opt_out).max())

    # per-kernel timing with HIP events on the launch stream, and the roofline of the dominant kernel
    with rt.Session(optimized, batch) as session:
        session.load_weights()
        session.set_input(x)
        ops = session.describe()
        op_ms = session.profile_ops(warmup=3, repeat=20)
    conv = [(op, ms) for op, ms in zip(ops, op_ms) if op['kind'] == 'conv_mfma']
    conv_flops = sum(op['flops'] for op, _ in conv)
    conv_ms = sum(ms for _, ms in conv)
    achieved = conv_flops / (conv_ms * 1e-3) / 1e12
    mem = [(op, ms) for op, ms in zip(ops, op_ms) if op['kind'] in ('pool', 'global_pool', 'nary', 'unary', 'conv_depthwise')]
    mem_gbs = (sum(op['bytes'] for op, _ in mem) / (sum(ms for _, ms in mem) * 1e-3) / 1e9) if mem else None
    roof_seq = network_roofline_ms(ops, parallel=False)
    roof_par = network_roofline_ms(ops, parallel=True)

    result = {
        'metric': 'batch-1 latency (ms) + images/s, Inception-v3 IOS dp_parallel schedule',
        'value': batch / (opt_wall * 1e-3),
        'unit': 'images/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': opt_wall,
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f32',
        'data': 'synthetic (N(0,1) input, seeded He-normal weights, zero bias)',
        'config': {'workload': f'inception_v3 3x299x299 batch {batch}, dp_parallel schedule (r=3, s=8), {args.executor} executor',
                   'global_batch': batch},
        'latency_ms': {'dp_parallel_wall': opt_wall, 'dp_parallel_events_mean': opt_ev, 'dp_parallel_events_min': opt_min,
                       'dp_parallel_events_std': opt_std, 'sequential_wall': seq_wall, 'sequential_events_mean': seq_ev,
                       'sequential_events_min': seq_min, 'sequential_events_std': seq_std},
        'speedup_vs_own_sequential': seq_wall / opt_wall,
        'max_abs_diff_between_schedules': schedule_diff,
        'search_seconds': search_s,
        'num_stages': sum(len(b.stages) for b in optimized.blocks),
        'network_roofline_ms': {'sequential': roof_seq, 'critical_path': roof_par,
                                'fraction_achieved': roof_par / opt_wall},
        'roofline': {'bound': 'mfma', 'kernel': 'conv_mfma_kernel (all 94 convolution launches of one pass)',
                     'achieved': achieved, 'peak': PEAK_FP32_MATRIX_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': achieved / PEAK_FP32_MATRIX_TFLOPS, 'traffic': None,
                     'flops_per_pass': conv_flops, 'kernel_ms_per_pass': conv_ms},
        'memory_bound_ops_gbs': mem_gbs,
        'device': device,
    }

    if args.sweep:
        sweep = {}
        for b in (16, 64):
            xb = np.random.default_rng(1).standard_normal((b, 3, 299, 299)).astype(np.float32)
            steps = max(10, args.steps // (b * 2))
            w_seq = timed_latency(graph, b, xb, steps, 3)[0]
            w_opt = timed_latency(optimized, b, xb, steps, 3)[0]
            sweep[str(b)] = {'sequential_ms': w_seq, 'dp_parallel_ms': w_opt, 'images_per_s': b / (min(w_seq, w_opt) * 1e-3)}
        result['batch_sweep'] = sweep

    if not args.no_cpu:
        import torch
        from oracle import ios_oracle
        threads = torch.get_num_threads()
        config, weights = graph.export_config(), ios_oracle.graph_weights(graph)
        ios_oracle.run_graph(config, weights, x)
        runs, t = 0, time.perf_counter()
        while runs < 6 or (time.perf_counter() - t < 10.0 and runs < 200):
            cpu_out = ios_oracle.run_graph(config, weights, x)
            runs += 1
        cpu_ms = (time.perf_counter() - t) / runs * 1e3
        err = np.abs(opt_out - cpu_out)
        result['cpu_baseline'] = {'value': batch / (cpu_ms * 1e-3), 'unit': 'images/s', 'cores': threads, 'kind': 'port',
                                  'sample': f'{runs} forward passes of the same graph, weights and input on the CPU oracle '
                                            f'(torch-CPU fp32, {threads} threads), {cpu_ms:.1f} ms each'}
        result['matches_cpu_oracle'] = bool((err <= 1e-4 + 1e-3 * np.abs(cpu_out)).all())
    print(json.dumps(result))


if __name__ == '__main__':
    main()
