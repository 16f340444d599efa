"""
Benchmark of the north-star path: Inception-v3 at batch 1 under the dp_parallel schedule found by the
dynamic-programming search with on-device stage measurements, on one MI355X.

A step is one forward pass over one synthetic batch (weights and input already resident in HBM).  Prints one
JSON line.  `roofline`: the convolution kernels of one pass, achieved = algorithmic FLOPs / HIP-event time of
their launches on the launch stream, against the fp32 matrix peak.  `cpu_baseline`: the CPU oracle on the same
graph, weights and input, timed on the host cores for about ten seconds.

Probe modes for the profiler (`--probe copy`, `--probe pass`) run a fixed small workload and print what the
counters should be compared with; they are used by the commands recorded under profiles/.
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
# HBM bytes per convolution launch of a batch-1 Inception-v3 pass, from FETCH_SIZE / WRITE_SIZE counter runs scaled by a
# copy kernel of known size (profiles/conv_kernel_hbm_traffic_inception_v3.md); counters cannot be read from inside this
# script, so the figure is the offline measurement of the same kernels.
MEASURED_CONV_TRAFFIC_BYTES_PER_LAUNCH = {1: 4.43e6, 64: 82.9e6}


def op_bound_ms(op):
    return max(op['flops'] / (PEAK_FP32_MATRIX_TFLOPS * 1e12), op['bytes'] / (PEAK_HBM_GBS * 1e9)) * 1e3


def network_roofline_ms(ops, parallel):
    """Sum over ops (or over stages of the slowest group) of max(flops / peak, bytes / bandwidth)."""
    if not parallel:
        return sum(op_bound_ms(op) for op in ops)
    stages = {}
    for op in ops:
        stages.setdefault(op['stage'], {}).setdefault(op['group'], 0.0)
        stages[op['stage']][op['group']] += op_bound_ms(op)
    return sum(max(groups.values()) for groups in stages.values())


def timed_latency(rt, np, graph, batch, x, steps, warmup):
    """Wall-clock ms per synchronised forward pass, event-timed latencies (reference protocol) and the output."""
    with rt.Session(graph, batch) as session:
        session.load_weights()
        session.set_input(x)
        for _ in range(warmup):
            session.run()
        t = time.perf_counter()
        for _ in range(steps):
            session.run()
        wall = (time.perf_counter() - t) / steps * 1e3
        events = session.measure(warmup=2, number=6, repeat=6)
        return {'wall': wall, 'events_mean': float(np.mean(events)), 'events_min': float(np.min(events)),
                'events_std': float(np.std(events))}, session.output()


def conv_roofline(rt, graph, batch, x, stages=False):
    """Per-kernel HIP-event timing of one pass; returns (ops, ms per op, conv summary, memory-bound GB/s[, stage ms])."""
    with rt.Session(graph, batch) as session:
        session.load_weights()
        session.set_input(x)
        ops = session.describe()
        op_ms = session.profile_ops(warmup=3, repeat=20)
        stage_ms = None
        if stages:
            repeat = 6
            _, per_stage = session.measure(warmup=2, number=6, repeat=repeat, profile_stage=True)
            count = len(per_stage) // repeat
            stage_ms = [sum(per_stage[r * count + i] for r in range(repeat)) / repeat for i in range(count)]
    conv = [(op, ms) for op, ms in zip(ops, op_ms) if op['kind'] == 'conv_mfma']
    flops = sum(op['flops'] for op, _ in conv)
    ms = sum(t for _, t in conv)
    mem = [(op, t) for op, t in zip(ops, op_ms) if op['kind'] in ('pool', 'global_pool', 'nary', 'unary', 'conv_depthwise')]
    mem_gbs = (sum(op['bytes'] for op, _ in mem) / (sum(t for _, t in mem) * 1e-3) / 1e9) if mem else None
    achieved = flops / (ms * 1e-3) / 1e12
    summary = {'bound': 'mfma', 'kernel': f'conv_kernel<...> ({len(conv)} convolution launches of one pass)',
               'achieved': achieved, 'peak': PEAK_FP32_MATRIX_TFLOPS, 'unit': 'TFLOP/s',
               'frac': achieved / PEAK_FP32_MATRIX_TFLOPS, 'traffic': MEASURED_CONV_TRAFFIC_BYTES_PER_LAUNCH.get(batch),
               'traffic_unit': 'bytes per launch (offline counter runs)',
               'algorithmic_bytes_per_launch': sum(op['bytes'] for op, _ in conv) / len(conv),
               'algorithmic_flops_per_launch': flops / len(conv), 'avg_launch_us': ms / len(conv) * 1e3,
               'flops_per_pass': flops, 'kernel_ms_per_pass': ms, 'launches': len(conv)}
    if stages:
        return ops, op_ms, summary, mem_gbs, stage_ms
    return ops, op_ms, summary, mem_gbs


def stage_overlap(ops, op_ms, stage_ms):
    """Multi-group stages: time of their operators launched one by one against the measured time of the stage."""
    groups, alone = {}, {}
    for op, ms in zip(ops, op_ms):
        if op['stage'] < 0:
            continue
        groups.setdefault(op['stage'], set()).add(op['group'])
        alone[op['stage']] = alone.get(op['stage'], 0.0) + ms
    multi = [s for s, g in groups.items() if len(g) > 1 and s < len(stage_ms)]
    if not multi:
        return None
    return {'multi_group_stages': len(multi), 'operators_one_by_one_ms': sum(alone[s] for s in multi),
            'stages_measured_ms': sum(stage_ms[s] for s in multi),
            'single_group_stages_ms': sum(ms for s, ms in enumerate(stage_ms) if s not in multi)}


def probe(args, np, ios, rt):
    """Small fixed workloads for counter collection."""
    rt.set_option('autotune', 1)
    if args.probe == 'copy':
        # y = relu(x) on 8 x 256 x 112 x 112: reads and writes 102,760,448 bytes per launch
        ios.reset_name()
        v = ios.placeholder((256, 112, 112))
        block = ios.Block(v.node)
        ios.relu(block, [[v]], is_exit=True)
        graph = ios.Graph('copy', v.node, [block])
        graph.sequential_schedule()
        x = np.random.default_rng(0).standard_normal((8, 256, 112, 112)).astype(np.float32)
        with rt.Session(graph, 8) as session:
            session.set_input(x)
            for _ in range(5):
                session.run()
            ms = session.profile_ops(1, 10)[0]
        nbytes = x.nbytes
        print(json.dumps({'probe': 'copy', 'kernel': 'nary_kernel', 'launches': 16, 'read_bytes_per_launch': nbytes,
                          'write_bytes_per_launch': nbytes, 'ms_per_launch': ms,
                          'gbs': 2 * nbytes / (ms * 1e-3) / 1e9}))
        return
    graph = ios.models.inception_v3(init_seed=0, init_scheme='he_normal')
    graph.sequential_schedule()
    x = np.random.default_rng(1).standard_normal((args.batch, 3, 299, 299)).astype(np.float32)
    rt.set_option('executor', 'streams')
    with rt.Session(graph, args.batch) as session:
        session.load_weights()
        session.set_input(x)
        for _ in range(3):
            session.run()
        ops = session.describe()
    conv = [op for op in ops if op['kind'] == 'conv_mfma']
    print(json.dumps({'probe': 'pass', 'batch': args.batch, 'passes': 3, 'schedule': 'sequential',
                      'conv_launches_per_pass': len(conv),
                      'conv_algorithmic_bytes_per_pass': sum(op['bytes'] for op in conv),
                      'conv_flops_per_pass': sum(op['flops'] for op in conv)}))


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
    parser.add_argument('--search', default='measured', choices=['measured', 'analytic'],
                        help="cost model of the schedule search: on-device stage measurements (default) or the "
                             "closed-form model (no device probes; keeps profiler traces small)")
    parser.add_argument('--search-number', type=int, default=6, help='passes per stage probe of the schedule search')
    parser.add_argument('--search-repeat', type=int, default=3, help='probes per candidate stage of the schedule search')
    parser.add_argument('--max-group-size', type=int, default=1,
                        help='pruning knob r of the schedule search (operators per group).  The fused executor runs the groups of a '
                             'stage level by level, so groups of one operator (r = 1) let the search place every level freely; the '
                             'reference default r = 3 is measured beside it')
    parser.add_argument('--max-num-groups', type=int, default=8, help='pruning knob s of the schedule search (groups per stage)')
    parser.add_argument('--search-restarts', type=int, default=2,
                        help='schedule searches to run (stage measurements are noisy: the schedule that measures faster as a whole is kept)')
    parser.add_argument('--no-sweep', action='store_true', help='skip the batch 16 / 64 sweep')
    parser.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    parser.add_argument('--no-configs', action='store_true', help='skip the other four configuration networks')
    parser.add_argument('--greedy-big', action='store_true',
                        help='use the greedy schedule for RandWire and NASNet instead of the measured search (half a minute each at r = 1, '
                             'minutes at r = 3)')
    parser.add_argument('--search-variants', action='store_true',
                        help="measured schedule search also for the reference table's large model variants (about two more minutes)")
    parser.add_argument('--option', action='append', default=[], metavar='KEY=VALUE', help='extra runtime option (repeatable)')
    parser.add_argument('--probe', choices=['copy', 'pass'], help='run a profiler probe instead of the benchmark')
    args = parser.parse_args()
    if args.gpus != 1:
        print('bench.py: this runtime is a single-GPU path; run with --gpus 1', file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import ios
    from ios.contrib import ios_runtime as rt

    if args.probe:
        probe(args, np, ios, rt)
        return

    device = rt.device_info()
    batch = args.batch
    graph = ios.models.inception_v3(init_seed=0, init_scheme='he_normal')
    x = np.random.default_rng(1).standard_normal((batch, 3, 299, 299)).astype(np.float32)

    # schedule search with measured stage latencies (not part of the timed steps)
    rt.set_option('autotune', 1)        # measure kernel configurations on first sight of a shape
    for item in args.option:
        key, _, value = item.partition('=')
        rt.set_option(key, value)
    rt.set_option('executor', args.search_executor)
    t0 = time.time()
    cost_model = ios.IOSCostModel() if args.search == 'measured' else ios.AnalyticCostModel()
    optimized, optimized_ms = None, None
    for _ in range(max(1, args.search_restarts if args.search == 'measured' else 1)):
        candidate = ios.optimize(graph, batch_size=batch, cost_model=cost_model, opt_type='dp_parallel', compute_weight=True,
                                 warmup=2, number=args.search_number, repeat=args.search_repeat,
                                 max_group_size=args.max_group_size, max_num_groups=args.max_num_groups)
        rt.set_option('executor', args.executor)
        candidate_ms = float(np.mean(rt.graph_latency(candidate, batch, warmup=2, number=6, repeat=6)))
        rt.set_option('executor', args.search_executor)
        if optimized is None or candidate_ms < optimized_ms:
            optimized, optimized_ms = candidate, candidate_ms
    search_s = time.time() - t0
    graph.sequential_schedule()

    rt.set_option('executor', args.executor)
    seq, seq_out = timed_latency(rt, np, graph, batch, x, args.steps, args.warmup)
    opt, opt_out = timed_latency(rt, np, optimized, batch, x, args.steps, args.warmup)

    # kernel roofline: every convolution in the configuration it runs with when it has the device to itself (the
    # sequential plan); inside the fused stage launches of the dp_parallel plan kernels cannot be timed one by one
    _, _, roofline, mem_gbs = conv_roofline(rt, graph, batch, x)
    ops, op_ms, _, _, stage_ms = conv_roofline(rt, optimized, batch, x, stages=True)
    roof_seq = network_roofline_ms(ops, parallel=False)
    roof_par = network_roofline_ms(ops, parallel=True)

    result = {
        'metric': 'batch-1 latency (ms) + images/s, Inception-v3 IOS dp_parallel schedule',
        'value': batch / (opt['wall'] * 1e-3),
        'unit': 'images/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': opt['wall'],
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f32',
        'data': 'synthetic (N(0,1) input, seeded He-normal weights, zero bias)',
        'config': {'workload': f'inception_v3 3x299x299 batch {batch}, dp_parallel schedule (r={args.max_group_size}, s={args.max_num_groups}), {args.executor} executor',
                   'global_batch': batch},
        'latency_ms': {'dp_parallel': opt, 'sequential': seq},
        'speedup_vs_own_sequential': seq['wall'] / opt['wall'],
        'max_abs_diff_between_schedules': float(np.abs(seq_out - opt_out).max()),
        'search_seconds': search_s,
        'num_stages': sum(len(b.stages) for b in optimized.blocks),
        'network_roofline_ms': {'sequential': roof_seq, 'critical_path': roof_par,
                                'fraction_of_critical_path_roofline': roof_par / opt['wall'],
                                'fraction_of_sequential_roofline': roof_seq / opt['wall']},
        'roofline': roofline,
        'memory_bound_ops_gbs': mem_gbs,
        'stage_overlap': stage_overlap(ops, op_ms, stage_ms),
        'device': {k: device[k] for k in ('name', 'arch', 'compute_units')},
    }

    # the same search with the reference's default pruning (r = 3, s = 8), for comparison with the headline's r and s
    if (args.max_group_size, args.max_num_groups) != (3, 8):
        rt.set_option('executor', args.search_executor)
        t0 = time.time()
        default_knobs = ios.optimize(graph, batch_size=batch, cost_model=cost_model, opt_type='dp_parallel', compute_weight=True,
                                     warmup=2, number=args.search_number, repeat=args.search_repeat)
        default_search_s = time.time() - t0
        graph.sequential_schedule()
        rt.set_option('executor', args.executor)
        r3, _ = timed_latency(rt, np, default_knobs, batch, x, args.steps, args.warmup)
        result['dp_parallel_r3_s8'] = {'latency_ms': r3, 'images_per_s': batch / (r3['wall'] * 1e-3), 'search_seconds': default_search_s,
                                       'num_stages': sum(len(b.stages) for b in default_knobs.blocks)}

    # the reference's best schedule family (parallel groups + merged convolutions, "IOS-Both"); the headline metric
    # is the dp_parallel schedule, this one is reported beside it
    rt.set_option('executor', args.search_executor)
    t0 = time.time()
    merged = ios.optimize(graph, batch_size=batch, cost_model=cost_model, opt_type='dp_parallel_merge', compute_weight=True,
                          warmup=2, number=args.search_number, repeat=args.search_repeat)
    merge_search_s = time.time() - t0
    graph.sequential_schedule()
    rt.set_option('executor', args.executor)
    both, both_out = timed_latency(rt, np, merged, batch, x, args.steps, args.warmup)
    result['dp_parallel_merge'] = {'latency_ms': both, 'images_per_s': batch / (both['wall'] * 1e-3), 'search_seconds': merge_search_s,
                                   'num_stages': sum(len(b.stages) for b in merged.blocks),
                                   'max_abs_diff_to_sequential': float(np.abs(seq_out - both_out).max())}

    if not args.no_sweep:
        sweep = {}
        for b in (16, 64):
            xb = np.random.default_rng(1).standard_normal((b, 3, 299, 299)).astype(np.float32)
            steps = max(10, args.steps // (b * 2))
            s_seq, out_seq = timed_latency(rt, np, graph, b, xb, steps, 3)
            s_opt, out_opt = timed_latency(rt, np, optimized, b, xb, steps, 3)
            # the schedule searched at this batch size (the reference's batch-size specialisation, experiments/specialization)
            rt.set_option('executor', args.search_executor)
            t0 = time.time()
            optimized_b = ios.optimize(graph, batch_size=b, cost_model=cost_model, opt_type='dp_parallel', compute_weight=True,
                                       warmup=2, number=args.search_number, repeat=args.search_repeat,
                                       max_group_size=args.max_group_size, max_num_groups=args.max_num_groups)
            search_b = time.time() - t0
            graph.sequential_schedule()
            rt.set_option('executor', args.executor)
            s_own, out_own = timed_latency(rt, np, optimized_b, b, xb, steps, 3)
            _, _, roof_b, _ = conv_roofline(rt, graph, b, xb)
            ops_b = rt.plan_describe(graph, b)
            best = min(s_seq['wall'], s_opt['wall'], s_own['wall'])
            sweep[str(b)] = {'sequential_ms': s_seq['wall'], 'dp_parallel_batch1_schedule_ms': s_opt['wall'],
                             'dp_parallel_ms': s_own['wall'], 'search_seconds': search_b,
                             'max_abs_diff_between_schedules': float(np.abs(out_seq - out_own).max()),
                             'images_per_s': b / (best * 1e-3),
                             'network_roofline_ms': network_roofline_ms(ops_b, parallel=False),
                             'fraction_of_network_roofline': network_roofline_ms(ops_b, parallel=False) / best,
                             'conv_tflops': roof_b['achieved'], 'conv_frac_of_fp32_matrix_peak': roof_b['frac']}
        result['batch_sweep'] = sweep
        # reduced-precision mode (bfloat16 operands, fp32 accumulation): not the headline metric, reported beside it
        rt.set_option('precision', 'bf16')
        reduced = {}
        for b in (1, 64):
            xb = np.random.default_rng(1).standard_normal((b, 3, 299, 299)).astype(np.float32)
            r_seq, out_b = timed_latency(rt, np, graph, b, xb, max(10, args.steps // (b * 2)), 3)
            reduced[str(b)] = {'sequential_ms': r_seq['wall'], 'images_per_s': b / (r_seq['wall'] * 1e-3)}
            if b == 1:
                reduced[str(b)]['max_abs_diff_to_fp32'] = float(np.abs(out_b - seq_out).max())
                reduced[str(b)]['fp32_output_scale'] = float(np.abs(seq_out).max())
        rt.set_option('precision', 'fp32')
        result['reduced_precision_bf16'] = reduced

    if not args.no_configs:
        configs = {}
        for name, make, search in (('sample_net', ios.models.sample_network, True),
                                   ('squeezenet_1_1', ios.models.squeezenet_1_1, True),
                                   ('randwire_small', ios.models.randwire_small, False),
                                   ('nasnet_mobile', ios.models.nasnet_mobile, False)):
            g = make(init_seed=0, init_scheme='he_normal')
            xc = np.random.default_rng(1).standard_normal((1, *g.enter_node.output_shape)).astype(np.float32)
            if search or not args.greedy_big:
                rt.set_option('executor', args.search_executor)
                t0 = time.time()
                scheduled = ios.optimize(g, batch_size=1, opt_type='dp_parallel', compute_weight=True, warmup=2, number=6, repeat=3,
                                         max_group_size=args.max_group_size, max_num_groups=args.max_num_groups)
                search_c = time.time() - t0
                label = 'dp_parallel'
                rt.set_option('executor', args.executor)
            else:   # --greedy-big
                scheduled = make(init_seed=0, init_scheme='he_normal')
                scheduled.greedy_schedule(4)
                label = 'greedy'
                search_c = 0.0
            g.sequential_schedule()
            c_seq, _ = timed_latency(rt, np, g, 1, xc, 100, 10)
            c_par, _ = timed_latency(rt, np, scheduled, 1, xc, 100, 10)
            ops_c = rt.plan_describe(g, 1)
            configs[name] = {'sequential_ms': c_seq['wall'], f'{label}_ms': c_par['wall'], 'search_seconds': search_c,
                             'network_roofline_ms': network_roofline_ms(ops_c, parallel=False)}
        result['other_configs_batch1'] = configs
        # the model variants the reference's own result table uses (its large RandWire / NASNet and SqueezeNet 1.0 with
        # bypass), sequential and greedy schedules: points of comparison with that table, not part of the metric
        variants = {}
        for name, make in (('squeezenet', ios.models.squeezenet), ('randwire_large', ios.models.randwire_large),
                           ('nasnet_large', ios.models.nasnet_large)):
            g = make(init_seed=0, init_scheme='he_normal')
            g.sequential_schedule()
            scheduled = make(init_seed=0, init_scheme='he_normal')
            scheduled.greedy_schedule(4)
            xc = np.random.default_rng(1).standard_normal((1, *g.enter_node.output_shape)).astype(np.float32)
            v_seq, _ = timed_latency(rt, np, g, 1, xc, 50, 5)
            v_par, _ = timed_latency(rt, np, scheduled, 1, xc, 50, 5)
            variants[name] = {'sequential_ms': v_seq['wall'], 'greedy_ms': v_par['wall']}
            if args.search_variants:
                rt.set_option('executor', args.search_executor)
                t0 = time.time()
                searched = ios.optimize(make(init_seed=0, init_scheme='he_normal'), batch_size=1, opt_type='dp_parallel', compute_weight=True,
                                        warmup=2, number=6, repeat=3, max_group_size=args.max_group_size, max_num_groups=args.max_num_groups)
                variants[name]['search_seconds'] = time.time() - t0
                rt.set_option('executor', args.executor)
                v_dp, _ = timed_latency(rt, np, searched, 1, xc, 50, 5)
                variants[name]['dp_parallel_ms'] = v_dp['wall']
        result['reference_table_variants_batch1'] = variants

    if not args.no_cpu:
        import torch
        from oracle import ios_oracle
        threads = torch.get_num_threads()
        config, weights = graph.export_config(), ios_oracle.graph_weights(graph)
        ios_oracle.run_graph(config, weights, x)
        runs, t = 0, time.perf_counter()
        while runs < 6 or (time.perf_counter() - t < 10.0 and runs < 2000):
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
