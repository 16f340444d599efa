"""
Benchmark of the north-star path: Inception-v3 at batch 1 under the dp_parallel schedule found by the
dynamic-programming search with on-device stage measurements, on one MI355X.

A step is one forward pass over one synthetic batch (weights and input already resident in HBM).  `ms_per_step` is the
latency of a pass under the reference's own timing protocol (`measure_latency`, src/ios/ios_runtime.cu:1419-1441): after W
warm-up passes, each of the K timed passes starts on an idle device (device synchronised first) and is bracketed by its own
pair of events; `ms_per_step` is their mean and `value` the images per second that latency allows.  The same K passes
queued back to back between two synchronisations (a throughput figure: the host's launch work overlaps the previous pass)
and with the host waiting for every pass are reported beside it as `throughput_ms_per_pass` and
`wall_host_waits_for_every_pass`.  Prints one JSON line.

`roofline` describes the kernel that takes the largest share of the timed pass: every launch of that pass (under the
executor that is timed) is issued back to back on the launch stream between two HIP events, launches are grouped by
kernel, and the dominant kernel's algorithmic FLOPs (or bytes) are divided by its time.  `kernels` lists the same
figures for every kernel of the pass.  `cpu_baseline`: the CPU oracle on the same graph, weights and input, timed on
the host cores for about ten seconds.  Every configuration network and every batch of the sweep is also compared with
the oracle under the strict tolerance |d| <= 1e-4 + 1e-3 |want|.

Probe modes for the profiler (`--probe copy | search | pass | floor`) run a fixed small workload and print what the counters
should be compared with; they are used by the commands recorded under profiles/.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for path in (ROOT, os.path.join(ROOT, 'inter-operator-scheduler_amd')):
    if path not in sys.path:
        sys.path.insert(0, path)

PEAK_FP32_MATRIX_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
# configuration networks: constructor name, initialisation (RandWire: batch norm folded into the convolutions, as its
# configuration says; the others seeded He-normal with zero bias)
CONFIG_MODELS = {'sample_net': ('sample_network', 'he_normal'), 'squeezenet_1_1': ('squeezenet_1_1', 'he_normal'),
                 'inception_v3': ('inception_v3', 'he_normal'), 'randwire_small': ('randwire_small', 'bn_folded'),
                 'nasnet_mobile': ('nasnet_mobile', 'he_normal')}
TRAFFIC_PROFILE = os.path.join(ROOT, 'profiles', 'hbm_traffic_by_kernel_inception_v3_batch1_dp_parallel.md')


def make_graph(ios, name):
    constructor, scheme = CONFIG_MODELS[name]
    return getattr(ios.models, constructor)(init_seed=0, init_scheme=scheme)


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


def progress(text):
    """A line on stderr per phase: a run that takes minutes says what it is doing (stdout carries the one JSON line)."""
    print(f'bench.py [{time.strftime("%H:%M:%S")}] {text}', file=sys.stderr, flush=True)


def timed_latency(rt, np, graph, batch, x, steps, warmup):
    """
    Latency of a forward pass, three ways over `steps` passes after `warmup` passes, and the output:
    `latency` - the reference protocol (device synchronised before every pass, an event pair around each, mean);
    `throughput_ms_per_pass` - wall clock over the passes queued back to back between two synchronisations (the device runs
    them one after the other, the host's launch work overlaps the previous pass);
    `wall_host_waits_for_every_pass` - wall clock with the host waiting for every pass.
    `events_*` repeat the reference protocol with the reference's default counts (warmup 2, number 6, repeat 6).
    """
    with rt.Session(graph, batch) as session:
        session.load_weights()
        session.set_input(x)
        latency = float(session.measure(warmup=warmup, number=steps, repeat=1)[0])
        session.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            session.enqueue()
        session.synchronize()
        queued = (time.perf_counter() - t) / steps * 1e3
        t = time.perf_counter()
        for _ in range(steps):
            session.run()
        wall_waiting = (time.perf_counter() - t) / steps * 1e3
        events = session.measure(warmup=2, number=6, repeat=6)
        return {'latency': latency, 'throughput_ms_per_pass': queued, 'wall_host_waits_for_every_pass': wall_waiting,
                'events_mean': float(np.mean(events)), 'events_min': float(np.min(events)),
                'events_std': float(np.std(events))}, session.output()


def oracle_check(np, got, want):
    """Strict tolerance of the path (rel 1e-3 / abs 1e-4, element by element) and how far the misses are."""
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    misses = int((err > 1e-4 + 1e-3 * np.abs(want.astype(np.float64))).sum())
    scale = float(np.abs(want).max())
    return {'matches_cpu_oracle': misses == 0, 'elements': int(want.size), 'elements_out_of_tolerance': misses,
            'max_abs_err': float(err.max()), 'output_scale': scale,
            'max_err_in_ulps_of_largest_output': float(err.max() / np.spacing(np.float32(scale)))}


def launch_profile(rt, graph, batch, x, stages=False):
    """
    Every launch of one pass under the executor in force, timed back to back with HIP events on the launch stream.
    Returns (ops, launches with 'ms', per-kernel totals[, per-stage ms of whole passes]).
    """
    with rt.Session(graph, batch) as session:
        session.load_weights()
        session.set_input(x)
        for _ in range(3):
            session.run()
        ops = session.describe()
        launches = session.launches()
        for launch, ms in zip(launches, session.profile_launches(warmup=3, repeat=20)):
            launch['ms'] = ms
        stage_ms = None
        if stages:
            repeat = 6
            _, per_stage = session.measure(warmup=2, number=6, repeat=repeat, profile_stage=True)
            count = len(per_stage) // repeat
            stage_ms = [sum(per_stage[r * count + i] for r in range(repeat)) / repeat for i in range(count)]
    kernels = {}
    for launch in launches:
        k = kernels.setdefault(launch['kernel'], {'launches': 0, 'ms': 0.0, 'flops': 0.0, 'matrix_flops': 0.0, 'bytes': 0.0})
        k['launches'] += 1
        for key in ('ms', 'flops', 'matrix_flops', 'bytes'):
            k[key] += launch[key]
    for k in kernels.values():
        k['tflops'] = k['matrix_flops'] / (k['ms'] * 1e-3) / 1e12
        k['gbs'] = k['bytes'] / (k['ms'] * 1e-3) / 1e9
        k['avg_launch_us'] = k['ms'] / k['launches'] * 1e3
        k['mfma_bound'] = k['matrix_flops'] / (PEAK_FP32_MATRIX_TFLOPS * 1e12) > k['bytes'] / (PEAK_HBM_GBS * 1e9)
    if stages:
        return ops, launches, kernels, stage_ms
    return ops, launches, kernels


def committed_traffic(kernel):
    """
    HBM bytes per launch of `kernel` and the provenance line of the committed counter summary they come from (an offline
    figure: FETCH_SIZE and WRITE_SIZE need a profiler run of their own).  A kernel the summary does not list is an error:
    the summary then describes another build and has to be collected again.
    """
    provenance = None
    with open(TRAFFIC_PROFILE) as f:
        for line in f:
            if line.startswith('Collected'):
                provenance = line.strip()
            match = re.match(r'\|\s*`([^`]+)`\s*\|(.*)\|\s*$', line)
            if match and match.group(1) == kernel:
                cells = [c.strip() for c in match.group(2).split('|')]
                return float(cells[-1]) * 1e6, provenance    # last column: traffic per launch, MB
    raise RuntimeError(f'{os.path.relpath(TRAFFIC_PROFILE, ROOT)} has no row for kernel {kernel}: collect the counters again')


def roofline_block(kernels, ms_per_step, headline=False):
    """The roofline object of the kernel with the largest share of the pass (counter traffic exists for the headline pass only)."""
    name, k = max(kernels.items(), key=lambda item: item[1]['ms'])
    if k['mfma_bound']:
        bound, achieved, peak, unit = 'mfma', k['tflops'], PEAK_FP32_MATRIX_TFLOPS, 'TFLOP/s'
    else:
        bound, achieved, peak, unit = 'hbm', k['gbs'], PEAK_HBM_GBS, 'GB/s'
    block = {'bound': bound, 'kernel': name, 'achieved': achieved, 'peak': peak, 'unit': unit, 'frac': achieved / peak,
             'traffic': None,
             'launches_per_pass': k['launches'], 'avg_launch_us': k['avg_launch_us'],
             'algorithmic_flops_per_launch': k['matrix_flops'] / k['launches'],
             'algorithmic_bytes_per_launch': k['bytes'] / k['launches'],
             'kernel_ms_per_pass': k['ms'], 'share_of_launch_time': k['ms'] / sum(v['ms'] for v in kernels.values()),
             'all_launches_ms_per_pass': sum(v['ms'] for v in kernels.values())}
    if headline:
        block['traffic'], provenance = committed_traffic(name)
        block['traffic_offline_counter_run'] = ('bytes per launch from FETCH_SIZE + WRITE_SIZE counter runs of a pass of this network, '
                                                'not of this run: ' + os.path.relpath(TRAFFIC_PROFILE, ROOT) + (' (' + provenance + ')' if provenance else ''))
    assert block['kernel_ms_per_pass'] <= ms_per_step, (block['kernel_ms_per_pass'], ms_per_step)
    return block


def memory_bound_ops(rt, graph, batch, x):
    """Achieved GB/s of the memory-bound operators of a pass, by kind (each launched back to back on one stream)."""
    rt.set_option('executor', 'streams')      # one launch per operator
    with rt.Session(graph, batch) as session:
        session.load_weights()
        session.set_input(x)
        ops = session.describe()
        op_ms = session.profile_ops(warmup=3, repeat=20)
    kinds = {}
    for op, ms in zip(ops, op_ms):
        if op['kind'] in ('pool', 'global_pool', 'nary', 'unary', 'conv_depthwise'):
            k = kinds.setdefault(op['kind'], {'launches': 0, 'ms': 0.0, 'bytes': 0.0})
            k['launches'] += 1
            k['ms'] += ms
            k['bytes'] += op['bytes']
    for k in kinds.values():
        k['gbs'] = k['bytes'] / (k['ms'] * 1e-3) / 1e9
        k['frac_of_hbm_peak'] = k['gbs'] / PEAK_HBM_GBS
    return kinds


def stage_overlap(ops, launches, stage_ms):
    """Multi-group stages: time of their operators' bounds and launches against the measured time of the stage."""
    groups = {}
    for op in ops:
        if op['stage'] >= 0:
            groups.setdefault(op['stage'], set()).add(op['group'])
    multi = [s for s, g in groups.items() if len(g) > 1 and s < len(stage_ms)]
    if not multi:
        return None
    return {'multi_group_stages': len(multi), 'stages_measured_ms': sum(stage_ms[s] for s in multi),
            'their_launches_back_to_back_ms': sum(l['ms'] for l in launches if l['stage'] in multi),
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
    if args.probe == 'layer':
        # one convolution with one pinned kernel configuration, a few launches: for counter runs on a single kernel
        ic, h, w, oc, kh, kw, stride, ph, pw = (int(v) for v in args.layer.split(','))
        rt.set_option('autotune', 0)
        rt.set_option('executor', 'streams')
        rt.set_option('conv_variant', rt.device_info()['conv_variants'].index(args.variant))
        rt.set_option('conv_split_k', args.split_k)
        ios.reset_name()
        v = ios.placeholder((ic, h, w))
        block = ios.Block(v.node)
        ios.conv2d(block, [[v]], oc, (kh, kw), (stride, stride), (ph, pw), 1, 'relu', is_exit=True)
        graph = ios.Graph('layer', v.node, [block])
        graph.init_weights(0, 'he_normal_bias')
        graph.sequential_schedule()
        x = np.random.default_rng(0).standard_normal((args.batch, ic, h, w)).astype(np.float32)
        with rt.Session(graph, args.batch) as session:
            session.load_weights()
            session.set_input(x)
            for _ in range(args.passes):
                session.run()
            ms = session.profile_ops(2, 10)[0]
            op = session.describe()[0]
        print(json.dumps({'probe': 'layer', 'layer': args.layer, 'batch': args.batch, 'variant': op.get('variant'), 'split_k': op.get('split_k'),
                          'us_per_launch': ms * 1e3, 'flops': op['flops'], 'bytes': op['bytes'],
                          'tflops': op['flops'] / (ms * 1e-3) / 1e12, 'gbs': op['bytes'] / (ms * 1e-3) / 1e9}))
        return
    if args.probe == 'floor':
        # what a launch costs when it does next to nothing: a chain of dependent tanh activations on one 8 x 8 x 8 tensor and a
        # chain of dependent 1x1 convolutions (8 -> 8 channels on 8 x 8 pixels), one launch each, under every executor
        results = {}
        for kind in ('activation', 'conv1x1'):
            ios.reset_name()
            v = ios.placeholder((8, 8, 8))
            block = ios.Block(v.node)
            t = v
            for i in range(args.floor_length):
                last = i == args.floor_length - 1
                if kind == 'activation':
                    t = ios.activation(block, [[t]], 'tanh', False, is_exit=last)
                else:
                    t = ios.conv2d(block, [[t]], 8, (1, 1), (1, 1), (0, 0), 1, 'tanh', is_exit=last)
            graph = ios.Graph('floor_' + kind, v.node, [block])
            graph.init_weights(0, 'he_normal_bias')
            graph.sequential_schedule()
            x = np.random.default_rng(0).standard_normal((1, 8, 8, 8)).astype(np.float32)
            for executor in args.floor_executors.split(','):
                rt.set_option('executor', executor)
                with rt.Session(graph, 1) as session:
                    session.load_weights()
                    session.set_input(x)
                    for _ in range(10):
                        session.run()
                    launches = len(session.launches())
                    session.synchronize()
                    t0 = time.perf_counter()
                    for _ in range(args.passes):
                        session.enqueue()
                    session.synchronize()
                    wall = (time.perf_counter() - t0) / args.passes * 1e3
                    events = float(np.min(session.measure(warmup=2, number=20, repeat=5)))
                results[f'{kind}/{executor}'] = {'launches_per_pass': launches, 'us_per_launch_queued_back_to_back': wall * 1e3 / launches,
                                                 'us_per_launch_event_timed': events * 1e3 / launches}
        print(json.dumps({'probe': 'floor', 'chain_length': args.floor_length, 'passes': args.passes, 'results': results}))
        return
    graph = make_graph(ios, args.model)
    batch = args.batch
    if args.probe == 'search':
        # measured schedule search (fills the kernel-configuration cache named by IOS_TUNE_CACHE), schedule written to a file
        rt.set_option('executor', args.search_executor)
        t0 = time.time()
        big = args.model in ('randwire_small', 'nasnet_mobile')      # (minutes at r = 3)
        group_size = args.big_max_group_size if big else args.max_group_size
        optimized = ios.optimize(graph, batch_size=batch, opt_type='dp_parallel', compute_weight=True, warmup=2,
                                 number=args.search_number, repeat=args.search_repeat,
                                 max_group_size=group_size, max_num_groups=args.max_num_groups)
        with open(args.schedule_file, 'w') as f:
            json.dump(optimized.export_config(), f)
        print(json.dumps({'probe': 'search', 'model': args.model, 'batch': batch, 'search_seconds': time.time() - t0,
                          'pruning': f'r = {group_size}, s = {args.max_num_groups}',
                          'stages': sum(len(b.stages) for b in optimized.blocks), 'schedule_file': args.schedule_file}))
        return
    # --probe pass: N passes of one plan and nothing else that launches kernels of the same names
    if args.schedule_file:
        with open(args.schedule_file) as f:
            scheduled = ios.Graph.from_config(json.load(f))
        scheduled.init_weights(0, CONFIG_MODELS[args.model][1])
        schedule = 'dp_parallel (from ' + os.path.basename(args.schedule_file) + ')'
    else:
        scheduled = graph
        scheduled.sequential_schedule()
        schedule = 'sequential'
    x = np.random.default_rng(1).standard_normal((batch, *graph.enter_node.output_shape)).astype(np.float32)
    rt.set_option('executor', args.executor)
    with rt.Session(scheduled, batch) as session:
        session.load_weights()
        session.set_input(x)
        for _ in range(args.passes):
            session.run()
        ops = session.describe()
        launches = session.launches()
    kernels = {}
    for launch in launches:
        k = kernels.setdefault(launch['kernel'], {'launches_per_pass': 0, 'flops_per_pass': 0.0, 'bytes_per_pass': 0.0})
        k['launches_per_pass'] += 1
        k['flops_per_pass'] += launch['flops']
        k['bytes_per_pass'] += launch['bytes']
    print(json.dumps({'probe': 'pass', 'model': args.model, 'batch': batch, 'passes': args.passes, 'schedule': schedule,
                      'executor': args.executor, 'kernels': kernels,
                      'launches': [{'stage': l['stage'], 'kernel': l['kernel'], 'blocks': l['blocks'], 'flops': l['flops'],
                                    'bytes': l['bytes'],
                                    'ops': [{'node': ops[i]['node'], 'kind': ops[i]['kind'], 'conv': ops[i].get('conv'),
                                             'out': ops[i]['out'], 'variant': ops[i].get('variant'), 'flops': ops[i]['flops'],
                                             'bytes': ops[i]['bytes']} for i in l['ops']]} for l in launches]}))


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
    parser.add_argument('--max-group-size', type=int, default=3,
                        help='pruning knob r of the schedule search (operators per group); 3 is the reference default '
                             '(python/ios/optimizer.py:42).  The search with r = 1 is measured beside it')
    parser.add_argument('--big-max-group-size', type=int, default=1,
                        help='r for the searches of RandWire and NASNet, whose searches take minutes at r = 3 (709 s / 168 s) and half a '
                             'minute at r = 1; their entries name the r they were searched with')
    parser.add_argument('--max-num-groups', type=int, default=8, help='pruning knob s of the schedule search (groups per stage)')
    parser.add_argument('--search-restarts', type=int, default=2,
                        help='schedule searches to run (stage measurements are noisy: the schedule that measures faster as a whole is kept)')
    parser.add_argument('--no-sweep', action='store_true', help='skip the batch 16 / 64 sweep')
    parser.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg and the oracle comparisons')
    parser.add_argument('--no-configs', action='store_true', help='skip the other four configuration networks')
    parser.add_argument('--no-extras', action='store_true',
                        help='skip the r = 1 and merged-convolution searches, the reduced-precision mode and the reference table variants')
    parser.add_argument('--greedy-big', action='store_true',
                        help='use the greedy schedule for RandWire and NASNet instead of the measured search')
    parser.add_argument('--search-variants', action='store_true',
                        help="also time the model variants of the reference's own result table (its large RandWire / NASNet, SqueezeNet 1.0 "
                             "with bypass, the chains and residual networks of its zoo) under sequential, greedy and searched schedules "
                             "(about three more minutes; not part of the metric)")
    parser.add_argument('--option', action='append', default=[], metavar='KEY=VALUE', help='extra runtime option (repeatable)')
    parser.add_argument('--probe', choices=['copy', 'search', 'pass', 'floor', 'layer'], help='run a profiler probe instead of the benchmark')
    parser.add_argument('--layer', default='80,73,73,192,3,3,1,0,0', help='probe layer: IC,H,W,OC,KH,KW,stride,pad_h,pad_w of the convolution')
    parser.add_argument('--variant', default='x3_m64n128_w2x2', help='probe layer: kernel configuration name')
    parser.add_argument('--split-k', type=int, default=1, help='probe layer: K slices')
    parser.add_argument('--model', default='inception_v3', choices=sorted(CONFIG_MODELS), help='network of the search / pass probes')
    parser.add_argument('--schedule-file', help='probe search: where to write the schedule; probe pass: schedule to run (default: sequential)')
    parser.add_argument('--passes', type=int, default=3, help='forward passes of the pass probe')
    parser.add_argument('--floor-length', type=int, default=50, help='floor probe: dependent operators in the chain')
    parser.add_argument('--floor-executors', default='streams,graph,fused,fused_graph',
                        help='floor probe: executors to time (graph replays are not traced by rocprofv3: give it streams,fused)')
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

    if not args.no_cpu:
        from oracle import ios_oracle

    device = rt.device_info()
    batch = args.batch
    graph = make_graph(ios, 'inception_v3')
    x = np.random.default_rng(1).standard_normal((batch, 3, 299, 299)).astype(np.float32)

    progress(f'schedule search, batch {batch}')
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
    progress('timed passes')
    seq, seq_out = timed_latency(rt, np, graph, batch, x, args.steps, args.warmup)
    opt, opt_out = timed_latency(rt, np, optimized, batch, x, args.steps, args.warmup)

    # the launches of the timed pass, under the executor that was timed
    ops, launches, kernels, stage_ms = launch_profile(rt, optimized, batch, x, stages=True)
    _, _, seq_kernels = launch_profile(rt, graph, batch, x)
    roof_seq = network_roofline_ms(ops, parallel=False)
    roof_par = network_roofline_ms(ops, parallel=True)
    conv_flops = sum(op['flops'] for op in ops if op['kind'] == 'conv_mfma')
    total_bytes = sum(op['bytes'] for op in ops)

    result = {
        'metric': 'batch-1 latency (ms) + images/s, Inception-v3 IOS dp_parallel schedule',
        'value': batch / (opt['latency'] * 1e-3),
        'unit': 'images/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': opt['latency'],
        'throughput_ms_per_pass': opt['throughput_ms_per_pass'],
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f32',
        'data': 'synthetic (N(0,1) input, seeded He-normal weights, zero bias)',
        'config': {'workload': f'inception_v3 3x299x299 batch {batch}, dp_parallel schedule (r={args.max_group_size}, s={args.max_num_groups}), {args.executor} executor',
                   'global_batch': batch},
        'latency_ms': {'dp_parallel': opt, 'sequential': seq},
        'speedup_vs_own_sequential': seq['latency'] / opt['latency'],
        'max_abs_diff_between_schedules': float(np.abs(seq_out - opt_out).max()),
        'search_seconds': search_s,
        'num_stages': sum(len(b.stages) for b in optimized.blocks),
        'launches_per_pass': len(launches),
        'network_roofline_ms': {'sequential': roof_seq, 'critical_path': roof_par,
                                'fraction_of_critical_path_roofline': roof_par / opt['latency'],
                                'fraction_of_sequential_roofline': roof_seq / opt['latency']},
        'whole_pass': {'matrix_tflops': conv_flops / (opt['latency'] * 1e-3) / 1e12,
                       'frac_of_fp32_matrix_peak': conv_flops / (opt['latency'] * 1e-3) / 1e12 / PEAK_FP32_MATRIX_TFLOPS,
                       'algorithmic_gbs': total_bytes / (opt['latency'] * 1e-3) / 1e9},
        'roofline': roofline_block(kernels, opt['latency'], headline=args.batch == 1),
        'kernels': kernels,
        'kernels_sequential_pass': seq_kernels,
        'stage_overlap': stage_overlap(ops, launches, stage_ms),
        'device': {k: device[k] for k in ('name', 'arch', 'compute_units')},
    }
    result['memory_bound_ops_gbs'] = memory_bound_ops(rt, graph, batch, x)
    rt.set_option('executor', args.executor)

    if not args.no_extras:
        # the same search with the other pruning of interest, for comparison with the headline's r and s: groups of one
        # operator (r = 1: the fused executor runs the groups of a stage level by level, so the search can cut every level
        # where it measures best) when the headline uses the reference's defaults, the reference's defaults otherwise
        other_r, other_s = (1, 8) if (args.max_group_size, args.max_num_groups) == (3, 8) else (3, 8)
        rt.set_option('executor', args.search_executor)
        t0 = time.time()
        other_knobs = ios.optimize(graph, batch_size=batch, cost_model=cost_model, opt_type='dp_parallel', compute_weight=True,
                                   warmup=2, number=args.search_number, repeat=args.search_repeat, max_group_size=other_r,
                                   max_num_groups=other_s)
        other_search_s = time.time() - t0
        graph.sequential_schedule()
        rt.set_option('executor', args.executor)
        other_ms, _ = timed_latency(rt, np, other_knobs, batch, x, args.steps, args.warmup)
        result[f'dp_parallel_r{other_r}_s{other_s}'] = {'latency_ms': other_ms, 'images_per_s': batch / (other_ms['latency'] * 1e-3),
                                                       'search_seconds': other_search_s,
                                                       'num_stages': sum(len(b.stages) for b in other_knobs.blocks)}

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
        result['dp_parallel_merge'] = {'latency_ms': both, 'images_per_s': batch / (both['latency'] * 1e-3), 'search_seconds': merge_search_s,
                                       'num_stages': sum(len(b.stages) for b in merged.blocks),
                                       'max_abs_diff_to_sequential': float(np.abs(seq_out - both_out).max())}

    if not args.no_sweep:
        sweep = {}
        for b in (16, 64):
            progress(f'batch {b}: sequential and batch-1 schedules')
            xb = np.random.default_rng(1).standard_normal((b, 3, 299, 299)).astype(np.float32)
            steps = max(30, args.steps // b)
            s_seq, out_seq = timed_latency(rt, np, graph, b, xb, steps, 3)
            s_opt, out_opt = timed_latency(rt, np, optimized, b, xb, steps, 3)
            # the schedule searched at this batch size (the reference's batch-size specialisation, experiments/specialization),
            # once for the fused executor and once for the graph executor, whose parallel branches launch every operator by
            # itself: there every kernel configuration competes for the parallel stages, also those too heavy on registers to
            # share a fused launch, which pays from batch 16 on
            searched = {}
            for executor, search_executor in ((args.executor, args.search_executor), ('graph', 'streams')):
                if executor in searched:
                    continue
                progress(f'batch {b}: schedule search for the {executor} executor')
                rt.set_option('executor', search_executor)
                t0 = time.time()
                candidate = ios.optimize(graph, batch_size=b, cost_model=cost_model, opt_type='dp_parallel', compute_weight=True,
                                         warmup=2, number=args.search_number, repeat=args.search_repeat,
                                         max_group_size=args.max_group_size, max_num_groups=args.max_num_groups)
                seconds = time.time() - t0
                graph.sequential_schedule()
                rt.set_option('executor', executor)
                timed, out = timed_latency(rt, np, candidate, b, xb, steps, 3)
                searched[executor] = {'schedule': candidate, 'timed': timed, 'out': out, 'search_seconds': seconds}
            own_executor = min(searched, key=lambda e: searched[e]['timed']['latency'])
            optimized_b, s_own, out_own = (searched[own_executor][k] for k in ('schedule', 'timed', 'out'))
            search_b = sum(v['search_seconds'] for v in searched.values())
            rt.set_option('executor', own_executor)
            _, _, kernels_b = launch_profile(rt, graph if s_seq['latency'] < s_own['latency'] else optimized_b, b, xb)
            ops_b = rt.plan_describe(graph, b)
            best = min(s_seq['latency'], s_opt['latency'], s_own['latency'])
            matrix_ms = sum(k['ms'] for k in kernels_b.values() if k['matrix_flops'] > 0)
            matrix_flops = sum(k['matrix_flops'] for k in kernels_b.values())
            sweep[str(b)] = {'sequential_ms': s_seq['latency'], 'dp_parallel_batch1_schedule_ms': s_opt['latency'],
                             'dp_parallel_ms': s_own['latency'], 'dp_parallel_executor': own_executor,
                             'dp_parallel_ms_by_executor': {e: v['timed']['latency'] for e, v in searched.items()},
                             'search_seconds': search_b,
                             'max_abs_diff_between_schedules': float(np.abs(out_seq - out_own).max()),
                             'images_per_s': b / (best * 1e-3),
                             'network_roofline_ms': network_roofline_ms(ops_b, parallel=False),
                             'fraction_of_network_roofline': network_roofline_ms(ops_b, parallel=False) / best,
                             'conv_tflops': matrix_flops / (matrix_ms * 1e-3) / 1e12,
                             'conv_frac_of_fp32_matrix_peak': matrix_flops / (matrix_ms * 1e-3) / 1e12 / PEAK_FP32_MATRIX_TFLOPS,
                             'roofline': roofline_block(kernels_b, best),
                             'memory_bound_ops_gbs': memory_bound_ops(rt, graph, b, xb)}
            rt.set_option('executor', args.executor)
            if not args.no_cpu:
                sample = sorted({0, b // 3, b - 1})      # an image's output depends on that image alone
                sweep[str(b)]['oracle'] = dict(oracle_check(np, out_own[sample], ios_oracle.run(graph, xb[sample])), images_checked=sample)
        result['batch_sweep'] = sweep
        if not args.no_extras:
            # reduced-precision modes (bfloat16 / half operands, fp32 accumulation): not the headline metric, reported beside it
            for precision in ('bf16', 'fp16'):
                rt.set_option('precision', precision)
                reduced = {}
                for b in (1, 64):
                    progress(f'{precision} operands, batch {b}')
                    xb = np.random.default_rng(1).standard_normal((b, 3, 299, 299)).astype(np.float32)
                    r_seq, out_b = timed_latency(rt, np, graph, b, xb, max(10, args.steps // (b * 2)), 3)
                    reduced[str(b)] = {'sequential_ms': r_seq['latency'], 'images_per_s': b / (r_seq['latency'] * 1e-3)}
                    if b == 1:
                        reduced[str(b)]['max_abs_diff_to_fp32'] = float(np.abs(out_b - seq_out).max())
                        reduced[str(b)]['fp32_output_scale'] = float(np.abs(seq_out).max())
                rt.set_option('precision', 'fp32')
                result['reduced_precision_' + precision] = reduced

    if not args.no_configs:
        configs = {}
        for name, search in (('sample_net', True), ('squeezenet_1_1', True), ('randwire_small', False), ('nasnet_mobile', False)):
            progress(f'{name}, batch 1')
            g = make_graph(ios, name)
            xc = np.random.default_rng(1).standard_normal((1, *g.enter_node.output_shape)).astype(np.float32)
            if search or not args.greedy_big:
                rt.set_option('executor', args.search_executor)
                t0 = time.time()
                # stages that are the same computation on the same shapes (NASNet's repeated cells) are measured once
                shared = ios.IOSCostModel(share_identical_stages=True)
                group_size = args.max_group_size if search else args.big_max_group_size
                scheduled = ios.optimize(g, batch_size=1, cost_model=shared, opt_type='dp_parallel', compute_weight=True, warmup=2, number=6,
                                         repeat=3, max_group_size=group_size, max_num_groups=args.max_num_groups)
                search_c = time.time() - t0
                label = 'dp_parallel'
                rt.set_option('executor', args.executor)
            else:   # --greedy-big
                scheduled = make_graph(ios, name)
                scheduled.greedy_schedule(4)
                label = 'greedy'
                search_c = 0.0
            other_ms = None
            if search and label == 'dp_parallel' and group_size != 1:
                # the small networks are searched in a fraction of a second: the r = 1 search beside the default one
                rt.set_option('executor', args.search_executor)
                single = ios.optimize(g, batch_size=1, cost_model=ios.IOSCostModel(share_identical_stages=True), opt_type='dp_parallel',
                                      compute_weight=True, warmup=2, number=6, repeat=3, max_group_size=1, max_num_groups=args.max_num_groups)
                rt.set_option('executor', args.executor)
                other_ms = timed_latency(rt, np, single, 1, xc, 100, 10)[0]['latency']
            g.sequential_schedule()
            c_seq, _ = timed_latency(rt, np, g, 1, xc, 100, 10)
            c_par, c_out = timed_latency(rt, np, scheduled, 1, xc, 100, 10)
            ops_c = rt.plan_describe(g, 1)
            _, launches_c, kernels_c = launch_profile(rt, scheduled, 1, xc)
            configs[name] = {'sequential_ms': c_seq['latency'], f'{label}_ms': c_par['latency'], 'search_seconds': search_c,
                             'search_pruning': None if label == 'greedy' else f'r={group_size}, s={args.max_num_groups}',
                             'initialisation': CONFIG_MODELS[name][1], 'device_operations': len(ops_c), 'launches_per_pass': len(launches_c),
                             'network_roofline_ms': network_roofline_ms(ops_c, parallel=False),
                             'fraction_of_network_roofline': network_roofline_ms(ops_c, parallel=False) / c_par['latency'],
                             'roofline': roofline_block(kernels_c, c_par['latency']),
                             'memory_bound_ops_gbs': memory_bound_ops(rt, g, 1, xc)}
            if other_ms is not None:
                configs[name]['dp_parallel_r1_ms'] = other_ms
            rt.set_option('executor', args.executor)
            if not args.no_cpu:
                configs[name]['oracle'] = oracle_check(np, c_out, ios_oracle.run(g, xc))
        result['other_configs_batch1'] = configs
        if args.search_variants:
            # the model variants the reference's own result table uses (its large RandWire / NASNet and SqueezeNet 1.0 with
            # bypass) and the chains / residual networks of its zoo, sequential and greedy schedules: points of comparison
            # with that table, not part of the metric
            variants = {}
            for name, make in (('squeezenet', ios.models.squeezenet), ('randwire_large', ios.models.randwire_large),
                               ('nasnet_large', ios.models.nasnet_large), ('alexnet', ios.models.alexnet), ('vgg_16', ios.models.vgg_16),
                               ('resnet18', ios.models.resnet18), ('resnet50', ios.models.resnet50)):
                g = make(init_seed=0, init_scheme='he_normal')
                g.sequential_schedule()
                scheduled = make(init_seed=0, init_scheme='he_normal')
                scheduled.greedy_schedule(4)
                xc = np.random.default_rng(1).standard_normal((1, *g.enter_node.output_shape)).astype(np.float32)
                v_seq, _ = timed_latency(rt, np, g, 1, xc, 50, 5)
                v_par, _ = timed_latency(rt, np, scheduled, 1, xc, 50, 5)
                variants[name] = {'sequential_ms': v_seq['latency'], 'greedy_ms': v_par['latency']}
                rt.set_option('executor', args.search_executor)
                t0 = time.time()
                searched = ios.optimize(make(init_seed=0, init_scheme='he_normal'), batch_size=1, opt_type='dp_parallel', compute_weight=True,
                                        warmup=2, number=6, repeat=3, max_group_size=args.big_max_group_size, max_num_groups=args.max_num_groups)
                variants[name]['search_seconds'] = time.time() - t0
                rt.set_option('executor', args.executor)
                v_dp, _ = timed_latency(rt, np, searched, 1, xc, 50, 5)
                variants[name]['dp_parallel_ms'] = v_dp['latency']
            result['reference_table_variants_batch1'] = variants

    if not args.no_cpu:
        progress('CPU baseline and oracle comparison')
        import torch
        threads = torch.get_num_threads()
        config, weights = graph.export_config(), ios_oracle.graph_weights(graph)
        ios_oracle.run_graph(config, weights, x)
        runs, t = 0, time.perf_counter()
        while runs < 6 or (time.perf_counter() - t < 10.0 and runs < 2000):
            cpu_out = ios_oracle.run_graph(config, weights, x)
            runs += 1
        cpu_ms = (time.perf_counter() - t) / runs * 1e3
        result['cpu_baseline'] = {'value': batch / (cpu_ms * 1e-3), 'unit': 'images/s', 'cores': threads, 'kind': 'port',
                                  'sample': f'{runs} forward passes of the same graph, weights and input on the CPU oracle '
                                            f'(torch-CPU fp32, {threads} threads), {cpu_ms:.1f} ms each'}
        result['oracle'] = oracle_check(np, opt_out, cpu_out)
        result['matches_cpu_oracle'] = result['oracle']['matches_cpu_oracle']
    print(json.dumps(result))


if __name__ == '__main__':
    main()
