"""The shared library loads without a GPU, exports every declared symbol and plans graphs on the host."""
import collections
import ctypes
import os
import re

import numpy as np
import pytest

import ios
from ios.contrib import ios_runtime as rt

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    with open(os.path.join(ROOT, 'include', 'ios_runtime.h')) as f:
        text = re.sub(r'/\*.*?\*/', '', f.read(), flags=re.S)
    return sorted(set(re.findall(r'\b(\w+)\s*\(', ' '.join(line for line in text.splitlines() if not line.startswith('#')))))


def test_library_exports_every_declared_symbol():
    lib = rt.get_lib()
    names = declared_symbols()
    assert {'graph_latency', 'block_latency', 'stage_latency', 'graph_inference', 'ios_last_error',
            'ios_session_create'} <= set(names)
    for name in names:
        assert getattr(lib, name) is not None, name


def test_missing_library_raises_file_not_found(monkeypatch):
    monkeypatch.setattr(rt, 'libname_list', ['nowhere/libios_runtime.so'])
    monkeypatch.delenv('IOS_RUNTIME_LIB', raising=False)
    with pytest.raises(FileNotFoundError, match='IOS Backend library not found'):
        rt.load_ios_library()


def test_host_planner_fuses_concats_and_folds_relus():
    graph = ios.models.inception_v3()
    graph.sequential_schedule()
    ops = rt.plan_describe(graph, 1)
    kinds = collections.Counter(op['kind'] for op in ops)
    # 94 convolutions, 13 window pools, 1 global pool and not a single copy: every concat is written in place
    assert kinds == {'conv_mfma': 94, 'pool': 13, 'global_pool': 1}
    by_node = {op['node']: op for op in ops}
    # conv '8' writes 64 channels into the 256-channel concat buffer of block 2: at batch 1 the stride is moot,
    # at batch 2 the batch stride must be that of the concat buffer
    ops2 = {op['node']: op for op in rt.plan_describe(graph, 2)}
    assert ops2['8']['out'] == [64, 35, 35] and ops2['8']['out_bstride'] == 256 * 35 * 35
    assert by_node['1']['conv']['sh'] == 2 and by_node['1']['out'] == [32, 149, 149]

    rw = ios.models.randwire_small()
    rw.sequential_schedule()
    ops = rt.plan_describe(rw, 1)
    kinds = collections.Counter(op['kind'] for op in ops)
    assert kinds['conv_depthwise'] == 96 and kinds['conv_mfma'] == 99
    # a node's depth-wise convolution adds the node's predecessors (and applies the ReLU) in its loader: the only summing
    # launches left are the stage outputs, the last of them inside the ReLU that follows it
    assert kinds['nary'] == 3 and kinds['unary'] == 0 and sum(kinds.values()) == 199
    depthwise = [op for op in ops if op['kind'] == 'conv_depthwise']
    assert max(op['inputs'] for op in depthwise) >= 5 and all(op['conv']['pre_relu'] for op in depthwise if op['inputs'] > 1)
    folded = [op for op in depthwise if op['inputs'] == 1 and op['conv']['pre_relu']]
    assert len(folded) > 0      # single-input nodes fold their ReLU into the depth-wise convolution
    nm = ios.models.nasnet_mobile()
    nm.sequential_schedule()
    ops = rt.plan_describe(nm, 1)
    assert len(ops) > 400
    # the sums of a cell's output concatenation are independent of each other: same unit, same level (one fused launch);
    # the 1x1 convolution of a separable unit follows its depth-wise convolution
    exit_sums = collections.defaultdict(list)
    for op in ops:
        if op['kind'] == 'nary':
            exit_sums[op['node']].append(op['level'])
    assert max(len(levels) for levels in exit_sums.values()) == 5 and all(set(levels) == {0} for levels in exit_sums.values())
    assert all(op['level'] == 1 for op in ops if op['kind'] == 'conv_mfma' and op['conv']['kh'] == 1 and ops[ops.index(op) - 1]['kind'] == 'conv_depthwise')


def test_host_planner_rejects_bad_documents():
    graph = ios.models.sample_network()
    with pytest.raises(RuntimeError, match='no schedule'):
        rt.plan_describe(graph, 1)
    graph.blocks[0].stages = [[['1'], ['4']], [['2'], ['3']], [['5']]]
    with pytest.raises(RuntimeError, match='not topological'):
        rt.plan_describe(graph, 1)
    graph.blocks[0].stages = [[['1']], [['2']], [['3']], [['5']]]
    with pytest.raises(RuntimeError, match="'5' runs before|missing"):
        rt.plan_describe(graph, 1)
    graph.sequential_schedule()
    config = graph.export_config()
    config['blocks'][0]['inner_nodes'][0]['type'] = 'softmax'
    doc = rt.c_string(__import__('json').dumps(config))
    assert rt.get_lib().ios_plan_describe(doc, 1, None, 0) == -1
    assert b'unsupported type softmax' in rt.get_lib().ios_last_error()
    with pytest.raises(RuntimeError):
        rt.plan_describe(graph, 0)


def test_host_planner_rejects_bad_operator_fields():
    """Geometry, channel counts and type names are checked before anything is sized or launched."""
    import copy
    import json
    graph = ios.models.squeezenet_1_1()
    graph.sequential_schedule()
    base = graph.export_config()

    def first_node_with(doc, field):
        for block in doc['blocks']:
            for node in block['inner_nodes'] + [block['exit_node']]:
                if field in node:
                    return node
        raise AssertionError(field)

    cases = [('stride', [0, 1], 'bad geometry'), ('kernel', [3, -3], 'bad geometry'), ('padding', [-1, 0], 'bad geometry'),
             ('padding', [1 << 20, 0], 'bad geometry'), ('groups', 0, 'not divisible by groups'), ('groups', 7, 'not divisible by groups'),
             ('out_channels', 0, 'channel'), ('out_channels', 10 ** 9, 'bad channel count'), ('pool_type', 'median', 'unknown pool_type'),
             ('act', 'gelu', 'unsupported activation')]
    for field, value, message in cases:
        doc = copy.deepcopy(base)
        first_node_with(doc, field)[field] = value
        assert rt.get_lib().ios_plan_describe(rt.c_string(json.dumps(doc)), 1, None, 0) == -1, (field, value)
        assert message.encode() in rt.get_lib().ios_last_error(), (field, value, rt.get_lib().ios_last_error())
    for shape in ([0, 224, 224], [3, -1, 224], [3, 224, 1 << 20]):
        doc = copy.deepcopy(base)
        doc['input']['output_shape'] = shape
        assert rt.get_lib().ios_plan_describe(rt.c_string(json.dumps(doc)), 1, None, 0) == -1, shape
        assert b'bad shape' in rt.get_lib().ios_last_error()
    doc = copy.deepcopy(base)
    doc['input']['output_shape'] = [3, 1e30, 224]      # a number no int can hold
    assert rt.get_lib().ios_plan_describe(rt.c_string(json.dumps(doc)), 1, None, 0) == -1
    assert b'out of integer range' in rt.get_lib().ios_last_error()
    for text in ('', '{', '{"name": 1}', 'null', '[]'):
        assert rt.get_lib().ios_plan_describe(rt.c_string(text), 1, None, 0) == -1, text


def test_json_reader_survives_hostile_documents():
    """A backslash as the last byte, a truncated \\u escape and absurd nesting are errors, not crashes."""
    lib = rt.get_lib()
    for text, message in (('{"name": "abc\\', b'unterminated string'), ('["\\', b'unterminated string'),
                          ('{"a\\u12', b'bad \\u escape'), ('["\\u', b'bad \\u escape'), ('["\\u00g0"]', b'bad \\u escape'),
                          ('[' * 100000, b'nesting deeper'), ('{"a":' * 70 + '1' + '}' * 70, b'nesting deeper'),
                          ('[' * 2000000, b'nesting deeper')):
        assert lib.ios_plan_describe(rt.c_string(text), 1, None, 0) == -1, text[:20]
        assert message in lib.ios_last_error(), (text[:20], lib.ios_last_error())
    # 60 levels are fine for the reader (the planner then rejects the document for its content)
    assert lib.ios_plan_describe(rt.c_string('[' * 60 + ']' * 60), 1, None, 0) == -1
    assert b'nesting' not in lib.ios_last_error()


def test_windows_larger_than_the_padded_input_are_rejected():
    """Truncating division would turn a window that does not fit into one output row: both sides refuse instead."""
    import copy
    import json
    ios.reset_name()
    v = ios.placeholder((4, 6, 6))
    block = ios.Block(v.node)
    ios.conv2d(block, [[v]], 4, (3, 3), (2, 2), (0, 0), is_exit=True)
    graph = ios.Graph('t', v.node, [block])
    graph.sequential_schedule()
    base = graph.export_config()
    assert len(rt.plan_describe(graph, 1)) == 1
    for shape in ([4, 2, 6], [4, 6, 2]):
        doc = copy.deepcopy(base)
        doc['input']['output_shape'] = shape
        assert rt.get_lib().ios_plan_describe(rt.c_string(json.dumps(doc)), 1, None, 0) == -1
        assert b'larger than the padded input' in rt.get_lib().ios_last_error()
    doc = copy.deepcopy(base)
    doc['input']['output_shape'] = [4, 2, 2]
    doc['blocks'][0]['exit_node'].update({'type': 'pool', 'pool_type': 'max'})
    assert rt.get_lib().ios_plan_describe(rt.c_string(json.dumps(doc)), 1, None, 0) == -1
    assert b'larger than the padded input' in rt.get_lib().ios_last_error()
    for build in (lambda b, x: ios.conv2d(b, [[x]], 4, (3, 3), (2, 2), (0, 0), is_exit=True),
                  lambda b, x: ios.pool2d(b, [[x]], 'max', (3, 3), (2, 2), (0, 0), is_exit=True)):
        ios.reset_name()
        small = ios.placeholder((4, 2, 2))
        with pytest.raises(ValueError, match='does not fit'):
            build(ios.Block(small.node), small)


def test_convolutions_of_parallel_stages_get_kernels_that_can_share_a_launch():
    """Host planner, closed-form kernel choice: every matrix-path convolution of a multi-group stage must be able
    to run inside a fused stage launch, at batch 1 and at a batch large enough for the LDS-tiled kernels."""
    import collections
    for batch in (1, 64):
        graph = ios.models.inception_v3()
        graph.greedy_schedule(8)
        ops = rt.plan_describe(graph, batch)
        groups = collections.defaultdict(set)
        for op in ops:
            groups[op['stage']].add(op['group'])
        shared = [op for op in ops if op['kind'] == 'conv_mfma' and len(groups[op['stage']]) > 1]
        alone = [op for op in ops if op['kind'] == 'conv_mfma' and len(groups[op['stage']]) == 1]
        assert len(shared) > 60 and alone
        assert all(op['fusable'] for op in shared), [op['variant'] for op in shared if not op['fusable']]
    # alone on the device at batch 64 the large layers take the LDS-tiled kernels, which are not fusable
    assert any(not op['fusable'] for op in alone)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    done = subprocess.run([sys.executable, os.path.join(root, 'bench.py'), '--gpus', '2'], capture_output=True, text=True, timeout=60)
    assert done.returncode != 0
    assert 'single-GPU' in done.stderr


def _simulate(ops):
    """Runs a plan symbolically: every float of the arena remembers the operation that wrote it last.  Returns, per
    operation, the writers it sees in what it reads; fails when two groups of one stage touch each other's memory."""
    # (`scratch`: the partial tiles of a split-K convolution, written and then read by that operation alone)
    ops = [dict(op, writes=op['writes'] + op.get('scratch', [])) for op in ops]
    end = max(r[1] for op in ops for key in ('writes', 'reads') for r in op[key])
    writer = np.full(end, -1, dtype=np.int32)
    seen = []
    stages = {}
    for index, op in enumerate(ops):
        stages.setdefault(op['stage'], []).append(index)
    for stage in sorted(stages):
        members = stages[stage]
        # concurrency inside the stage: what one group writes, no other group reads or writes
        mark = {}
        for index in members:
            for begin, stop in ops[index]['writes']:
                mark.setdefault(ops[index]['group'], []).append((begin, stop))
        for index in members:
            op = ops[index]
            for group, ranges in mark.items():
                if group == op['group']:
                    continue
                for begin, stop in ranges:
                    for b, e in op['reads'] + op['writes']:
                        assert e <= begin or stop <= b, (op['node'], 'overlaps group', group, 'in stage', stage)
        for index in members:       # launch order inside a stage: groups one after the other is one valid order
            op = ops[index]
            found = set()
            for begin, stop in op['reads']:
                found.update(np.unique(writer[begin:stop]).tolist())
            seen.append(tuple(sorted(found)))
            for begin, stop in op['writes']:
                writer[begin:stop] = index
    return seen


@pytest.mark.parametrize('name,batch,schedule', [('squeezenet_1_1', 2, 'sequential'), ('squeezenet_1_1', 1, 'greedy'),
                                                 ('randwire_small', 1, 'greedy'), ('nasnet_mobile', 1, 'greedy'),
                                                 ('nasnet_mobile', 2, 'sequential'), ('inception_v3', 1, 'greedy'),
                                                 ('resnet50', 1, 'greedy'), ('resnet18', 2, 'sequential')])
def test_arena_reuse_never_lets_an_operator_read_what_another_overwrote(name, batch, schedule):
    graph = getattr(ios.models, name)()
    if schedule == 'greedy':
        graph.greedy_schedule(8)
    else:
        graph.sequential_schedule()
    try:
        rt.set_option('arena_reuse', 0)
        plain = rt.plan_describe(graph, batch)
        plain_bytes = rt.plan_arena_bytes(graph, batch)
        rt.set_option('arena_reuse', 1)
        shared = rt.plan_describe(graph, batch)
        shared_bytes = rt.plan_arena_bytes(graph, batch)
    finally:
        rt.set_option('arena_reuse', 1)
    assert [(op['node'], op['kind']) for op in plain] == [(op['node'], op['kind']) for op in shared]
    assert shared_bytes < 0.9 * plain_bytes
    # every operation reads values written by exactly the same operations (or by nobody: the input, filters) in both plans
    assert _simulate(shared) == _simulate(plain)
    # the network input is never overwritten: no operation writes where the first operation reads
    first_reads = shared[0]['reads']
    for op in shared:
        for begin, stop in op['writes']:
            assert all(e <= begin or stop <= b for b, e in first_reads), op['node']


@pytest.mark.parametrize('tiles,split', [(1, 2), (5, 3), (8, 4), (9, 2), (48, 4), (190, 2), (231, 5), (1000, 16), (7, 64)])
def test_xcd_local_split_k_numbering(tiles, split):
    """The grid of a split-K convolution whose slices meet inside one XCD: every (tile, slice) exactly once, all slices of a
    tile on blocks with the same index modulo 8 (the dispatcher deals workgroups to the 8 XCDs round-robin), every residue
    class owning a contiguous range of tiles of nearly equal length, idle blocks only where a class has one tile less."""
    lib = rt.get_lib()
    blocks = lib.ios_xcd_numbering(tiles, split, None, None, 0)
    assert blocks == 8 * ((tiles + 7) // 8) * split
    tile = (ctypes.c_int * blocks)()
    piece = (ctypes.c_int * blocks)()
    assert lib.ios_xcd_numbering(tiles, split, tile, piece, blocks) == blocks
    seen = {}
    for block in range(blocks):
        if tile[block] < 0:
            continue
        assert 0 <= tile[block] < tiles and 0 <= piece[block] < split
        assert (tile[block], piece[block]) not in seen
        seen[(tile[block], piece[block])] = block
    assert len(seen) == tiles * split
    per_class = {}
    for (t, _), block in seen.items():
        per_class.setdefault(block % 8, set()).add(t)
    for t in range(tiles):
        assert len({seen[(t, z)] % 8 for z in range(split)}) == 1       # one XCD per tile
        order = [seen[(t, z)] for z in range(split)]
        assert order == sorted(order) and order[-1] - order[0] == 8 * (split - 1)   # dispatched together, slice 0 first
    sizes = [len(per_class.get(c, ())) for c in range(8)]
    assert max(sizes) - min(sizes) <= 1 and sum(sizes) == tiles
    for c, owned in per_class.items():
        assert sorted(owned) == list(range(min(owned), max(owned) + 1))  # contiguous: an XCD's L2 sees neighbouring tiles
    assert blocks - len(seen) == (8 * ((tiles + 7) // 8) - tiles) * split


def test_three_bfloat16_terms_of_an_fp32_value_are_exact():
    """The x3_* convolution kernels multiply fp32 operands on the bfloat16 matrix pipe: x = hi + mid + lo with three bfloat16
    terms must hold exactly (it is what makes six bfloat16 products as accurate as one fp32 product)."""
    lib = rt.get_lib()
    lib.ios_split_bf16x3.argtypes = [ctypes.c_float, ctypes.POINTER(ctypes.c_uint)]
    lib.ios_split_bf16x3.restype = None
    rng = np.random.default_rng(7)
    values = np.concatenate([rng.standard_normal(4000).astype(np.float32) * np.float32(10.0) ** rng.integers(-20, 20, 4000).astype(np.float32),
                             np.array([0.0, -0.0, 1.0, -1.0, 1.0 + 2.0 ** -23, 1.0 - 2.0 ** -24, 3.4028235e38, -3.4028235e38, 1.17549435e-38,
                                       0.1, 1 / 3, 255.99998, 65535.996, 2.0 ** -100 * 1.9999999], dtype=np.float32)])
    terms = (ctypes.c_uint * 3)()
    for x in values:
        lib.ios_split_bf16x3(ctypes.c_float(float(x)), terms)
        parts = np.array(list(terms), dtype=np.uint32)
        assert not (parts & 0xffff).any()                       # each term is a bfloat16
        as_float = parts.view(np.float32).astype(np.float64)
        assert as_float.sum() == np.float64(x), (x, as_float)
        assert abs(as_float[1]) <= abs(as_float[0]) * 2.0 ** -7 + 0 and abs(as_float[2]) <= abs(as_float[0]) * 2.0 ** -15 + 0


def test_split_k_partial_tiles_share_the_arena_like_any_other_region():
    # every convolution forced to four K slices: their partial tiles are regions with a lifetime of one stage, so they share
    # addresses with tensors that are dead by then, and must never land on one that a later operation still reads
    graph = ios.models.inception_v3()
    graph.greedy_schedule(8)
    try:
        rt.set_option('host_plan_split_k', 4)
        rt.set_option('arena_reuse', 0)
        plain = rt.plan_describe(graph, 2)
        rt.set_option('arena_reuse', 1)
        shared = rt.plan_describe(graph, 2)
    finally:
        rt.set_option('host_plan_split_k', 0)
        rt.set_option('arena_reuse', 1)
    with_scratch = [op for op in shared if op.get('scratch')]
    assert len(with_scratch) > 50 and all(op['split_k'] == 4 for op in with_scratch)
    assert _simulate(shared) == _simulate(plain)
    # the partial tiles do share addresses with operator outputs in the reusing plan (the test above would be vacuous otherwise)
    outputs = [r for op in shared for r in op['writes']]
    assert any(b < e2 and b2 < e for op in with_scratch for b, e in op['scratch'] for b2, e2 in outputs)


def test_residual_additions_join_the_activation_behind_them_and_pool_names_follow_the_reference():
    # ResNet-50: 16 residual units end in convolution, addition of the skip value, in-place ReLU (reference
    # python/ios/models/resnet.py:19-27).  The convolution's epilogue adds the skip value and applies the ReLU: one launch for
    # the three operators, no tensor for the convolution and the addition
    graph = ios.models.resnet50()
    ops = rt.plan_describe(graph, 1)
    kinds = [op['kind'] for op in ops]
    assert kinds.count('conv_mfma') == 53 and kinds.count('pool') == 1 and len(ops) == 54
    residual = [op for op in ops if op.get('residual')]
    nodes = {n.name: n for n in graph.nodes()}
    assert len(residual) == 16 and all(op['post_relu'] == 1 and len(op['reads']) == 2 and nodes[op['node']].act == 'identity' for op in residual)
    # ResNet-18 / 34 have no activation behind their additions
    ops18 = rt.plan_describe(ios.models.resnet18(), 1)
    assert len(ops18) == 21 and sum(1 for op in ops18 if op.get('residual') and op['post_relu'] == 0) == 8
    # the skip value has to be complete before the convolution starts: with the projection '3' scheduled beside the last
    # convolution '6' of the first unit, the addition stays a launch of its own (the ReLU behind it still joins it)
    late = ios.models.resnet50()
    stages = late.blocks[1].stages
    assert stages[:5] == [[['3']], [['4']], [['5']], [['6']], [['7']]]
    late.blocks[1].stages = [[['4']], [['5']], [['6'], ['3']]] + stages[4:]
    ops_late = rt.plan_describe(late, 1)
    assert sum(1 for op in ops_late if op.get('residual')) == 15
    kept = [op for op in ops_late if op['kind'] == 'nary']
    assert len(kept) == 1 and kept[0]['node'] == '8' and kept[0]['act'] == 1 and len(kept[0]['reads']) == 2
    # in one group the later of the two convolutions adds the earlier one's output, whichever it is
    for order, adder in ((['6', '3'], '3'), (['3', '6'], '6')):
        late.blocks[1].stages = [[['4']], [['5']], [order]] + stages[4:]
        found = [op['node'] for op in rt.plan_describe(late, 1) if op.get('residual')]
        assert len(found) == 16 and found[0] == adder
    # pooling names: the reference looks for the substrings "max" and "global" (src/ios/ios_runtime.cu:1047-1051) and its
    # AlexNet writes 'max_pool'
    config = ios.models.alexnet().export_config()
    plain = rt.plan_describe(ios.Graph.from_config(config), 1)
    for node in config['blocks'][0]['inner_nodes']:
        if node['type'] == 'pool':
            node['pool_type'] = 'max_pool'
    renamed = rt.plan_describe(ios.Graph.from_config(config), 1)
    assert [(op['kind'], op['reads'], op['writes']) for op in renamed] == [(op['kind'], op['reads'], op['writes']) for op in plain]


@pytest.mark.parametrize('seed', range(0, 120, 3))
def test_random_networks_plan_and_share_the_arena_safely(seed):
    """Random wiring of every operator kind under random schedules (tests/random_graphs.py): the planner accepts them, and
    with arena reuse every operation still reads what the same operations wrote."""
    import random_graphs
    graph, batch, _ = random_graphs.random_graph(seed)
    try:
        rt.set_option('arena_reuse', 0)
        plain = rt.plan_describe(graph, batch)
        rt.set_option('arena_reuse', 1)
        shared = rt.plan_describe(graph, batch)
    finally:
        rt.set_option('arena_reuse', 1)
    assert [(op['node'], op['kind']) for op in plain] == [(op['node'], op['kind']) for op in shared]
    assert _simulate(shared) == _simulate(plain)
    assert rt.plan_arena_bytes(graph, batch) > 0


def test_planner_options_need_no_device_and_change_the_plan():
    graph = ios.models.inception_v3()
    graph.sequential_schedule()
    try:
        first = rt.plan_describe(graph, 16)[0]
        assert first['kind'] == 'conv_direct' and first['thin'] is True      # 16 x 149 x 149 output pixels: the first-layer kernel
        assert rt.plan_describe(graph, 1)[0]['kind'] == 'conv_mfma'           # batch 1: the matrix path
        rt.set_option('thin_conv_min_pixels', -1)
        assert rt.plan_describe(graph, 16)[0]['kind'] == 'conv_mfma'
        rt.set_option('thin_conv_min_pixels', 0)
        assert rt.plan_describe(graph, 1)[0]['kind'] == 'conv_direct'
        # only 3 x 3 convolutions of 3-channel inputs qualify
        assert sum(op['kind'] == 'conv_direct' for op in rt.plan_describe(graph, 1)) == 1
        rt.set_option('arena_reuse', 0)
        plain = rt.plan_arena_bytes(graph, 16)
        rt.set_option('arena_reuse', 1)
        assert rt.plan_arena_bytes(graph, 16) < plain
    finally:
        rt.set_option('thin_conv_min_pixels', 1 << 18)
        rt.set_option('arena_reuse', 1)


def test_average_pools_change_places_with_the_pointwise_convolution_behind_them():
    """
    Inception's pool branches (reference python/ios/models/inception_v3.py:28-29,62-63,96-97): the launch at the pool's place
    is the 1 x 1 convolution without bias and activation, the launch at the convolution's place pools its output and finishes
    it; the pooled input tensor no longer exists.  Pools that change the map size, max pools and pools with other readers stay.
    """
    graph = ios.models.inception_v3()
    graph.sequential_schedule()
    by_name = {node.name: node for node in graph.nodes()}
    try:
        ops = rt.plan_describe(graph, 2)
        linear = [op for op in ops if op.get('linear')]
        finishing = [op for op in ops if 'adds_bias_of' in op]
        assert len(linear) == len(finishing) == 9
        for conv_op, pool_op in zip(linear, finishing):
            pool_node, conv_node = by_name[conv_op['node']], by_name[pool_op['node']]
            assert pool_node.type == 'pool' and conv_node.type == 'conv' and pool_op['adds_bias_of'] == conv_node.name
            assert conv_op['kind'] == 'conv_mfma' and conv_op['conv']['act'] == 0 and pool_op['kind'] == 'pool'
            assert conv_op['stage'] < pool_op['stage']
            # z has the convolution's channels on the pool's input map; the pool writes the convolution's tensor
            assert conv_op['out'] == [conv_node.out_channels, *pool_node.output_shape[1:]]
            assert pool_op['out'] == list(conv_node.output_shape) and pool_op['act'] == 1
            assert conv_op['writes'] == pool_op['reads']
        assert sum(op['kind'] in ('pool', 'global_pool') for op in ops) == 14
        _simulate(ops)
        rt.set_option('commute_pool_conv', 0)
        plain = rt.plan_describe(graph, 2)
        assert not any(op.get('linear') or 'adds_bias_of' in op for op in plain)
        assert sum(op["bytes"] for op in ops) < 0.95 * sum(op['bytes'] for op in plain)
    finally:
        rt.set_option('commute_pool_conv', 1)
    # NASNet's reductions pool with stride 2 in front of 1 x 1 convolutions: the convolution would see four times the pixels
    nasnet = ios.models.nasnet_mobile()
    nasnet.sequential_schedule()
    assert not any(op.get('linear') for op in rt.plan_describe(nasnet, 1))
