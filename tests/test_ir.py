"""Host-side IR, builder API, wire format and model zoo."""
import json
import os

import numpy as np
import pytest

import ios
from ios.ir import Conv, Graph, Identity, Pool, Sequential, Value

GOLDEN = os.path.join(os.path.dirname(__file__), 'golden')


def test_sample_network_shapes_and_pretty_print():
    graph = ios.models.sample_network()
    assert tuple(graph.exit_node.output_shape) == (1875, 15, 15)    # README output shape
    graph.sequential_schedule()
    # text printed by the reference README for the sequential schedule of this network
    assert str(graph) == ("Sequential(\n  [1]Conv2d(0)\n  [2]Conv2d(0)\n  [3]Conv2d(0)\n  [4]Conv2d(1)\n"
                          "  [5]Concat(4,2,3)\n)")
    graph.blocks[0].stages = [[['1'], ['2']], [['4'], ['3']], [['5']]]
    assert str(graph) == ("Sequential(\n  Parallel(\n    [1]Conv2d(0)\n    [2]Conv2d(0)\n  )\n  Parallel(\n"
                          "    [4]Conv2d(1)\n    [3]Conv2d(0)\n  )\n  [5]Concat(4,2,3)\n)")


def test_inception_v3_topology():
    graph = ios.models.inception_v3()
    nodes = list(graph.nodes())
    assert [n.name for n in nodes] == [str(i) for i in range(120)]
    assert len(graph.blocks) == 13
    assert len(graph.conv_nodes()) == 94
    assert sum(isinstance(n, Pool) for n in nodes) == 14
    assert sum(isinstance(n, Identity) for n in nodes) == 11
    by_name = {n.name: n for n in nodes}
    # spatial sizes of the stem: 149, 147, 147, 73, 73, 71, 35
    assert [by_name[str(i)].output_shape[1] for i in range(1, 8)] == [149, 147, 147, 73, 73, 71, 35]
    exits = [tuple(b.exit_node.output_shape) for b in graph.blocks]
    assert exits == [(192, 35, 35), (256, 35, 35), (288, 35, 35), (288, 35, 35), (768, 17, 17), (768, 17, 17),
                     (768, 17, 17), (768, 17, 17), (768, 17, 17), (1280, 8, 8), (2048, 8, 8), (2048, 8, 8),
                     (2048, 1, 1)]
    macs = sum(np.prod(c.output_shape) * c.fan_in for c in graph.conv_nodes())
    assert macs == pytest.approx(5.711e9, rel=2e-3)
    weights = sum(np.prod(c.weight_shape) for c in graph.conv_nodes()) * 4
    assert weights == pytest.approx(87.07e6, rel=2e-3)


def test_inception_schedule_fixture_round_trip():
    # a schedule document of the shape the reference exports for an optimised Inception-v3 (merged convs,
    # channel-slice inputs, multi-group stages); it was produced by this package's optimizer
    with open(os.path.join(GOLDEN, 'inception_v3_dp_parallel_merge.json')) as f:
        config = json.load(f)
    graph = Graph.from_config(config)
    assert json.loads(json.dumps(graph.export_config())) == config
    assert tuple(graph.exit_node.output_shape) == (2048, 1, 1)
    plain = {n.name: n for n in ios.models.inception_v3().nodes()}
    seen = set()
    for node in graph.nodes():
        seen.update(node.hint_name.split())
        if ' ' not in node.hint_name and node.name in plain and node.type == 'conv':
            ref = plain[node.name]
            assert (node.out_channels, tuple(node.kernel), tuple(node.stride), tuple(node.padding)) == \
                   (ref.out_channels, tuple(ref.kernel), tuple(ref.stride), tuple(ref.padding))
    assert seen == {str(i) for i in range(120)}


@pytest.mark.parametrize('name', ['1', '16', '32', '64', '128', 'k80', 'v100'])
def test_reference_schedule_files_load_round_trip_and_plan(name):
    """
    The reference's own schedule files (experiments/specialization/schedules/*.json, committed as fixtures): they load,
    export back to the identical document, name the plain model's operators, and the host planner accepts them.
    """
    import reference_schedules
    from ios.contrib import ios_runtime as rt
    config = reference_schedules.load_config(name)
    graph = Graph.from_config(config)
    assert json.loads(json.dumps(graph.export_config())) == config
    assert tuple(graph.enter_node.output_shape) == (3, 299, 299) and tuple(graph.exit_node.output_shape) == (2048, 1, 1)
    plain = {n.name: n for n in ios.models.inception_v3().nodes()}
    tokens = []
    for node in graph.nodes():
        tokens += node.hint_name.split()
        if ' ' in node.hint_name:
            assert node.type == 'conv' and node.out_channels == sum(plain[t].out_channels for t in node.hint_name.split())
            continue
        ref = plain[node.name]
        assert node.type == ref.type and tuple(node.output_shape) == tuple(ref.output_shape) and node.hint_name == ref.hint_name
        if node.type == 'conv':
            assert (node.out_channels, tuple(node.kernel), tuple(node.stride), tuple(node.padding), node.groups, node.act) == \
                   (ref.out_channels, tuple(ref.kernel), tuple(ref.stride), tuple(ref.padding), ref.groups, ref.act)
        if node.type == 'pool':
            assert (node.pool_type, tuple(node.kernel), tuple(node.stride), tuple(node.padding)) == \
                   (ref.pool_type, tuple(ref.kernel), tuple(ref.stride), tuple(ref.padding))
    # every operator of the plain model (placeholder 0, operators 1..119) appears exactly once, merged or not
    assert sorted(tokens, key=int) == [str(i) for i in range(120)]
    scheduled = sorted(n for block in graph.blocks for stage in block.stages for group in stage for n in group)
    assert scheduled == sorted(n.name for n in graph.nodes() if n is not graph.enter_node)
    ops = rt.plan_describe(graph, reference_schedules.TUNED_BATCH[name])
    # slices of merged convolutions are read in place by convolutions and pools; only a slice that is itself a term of a
    # block's concatenation is copied there (at most one per merged convolution)
    # (at the batch sizes 16 ... 128 the first layer, a 3 x 3 convolution of the 3-channel image, takes the direct kernel)
    assert {op['kind'] for op in ops} <= {'conv_mfma', 'conv_direct', 'pool', 'global_pool', 'unary'}
    assert [op['kind'] for op in ops].count('conv_direct') <= 1
    merged = sum(' ' in n.hint_name for n in graph.nodes())
    assert sum(op['kind'] == 'unary' for op in ops) <= merged
    assert sum(op['kind'] in ('conv_mfma', 'conv_direct') for op in ops) == sum(n.type == 'conv' for n in graph.nodes())


def test_reference_schedule_weights_from_the_plain_model_reproduce_its_output_on_the_oracle():
    """Stacked weights of the merged convolutions (reference optimizer.py:662-711): same network function."""
    import reference_schedules
    from oracle import ios_oracle
    plain = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    plain.sequential_schedule()
    x = np.random.default_rng(2).standard_normal((1, 3, 299, 299)).astype(np.float32)
    want = ios_oracle.run(plain, x)
    for name in ('1', '64'):
        graph = reference_schedules.load(name)
        reference_schedules.adopt_weights(graph, plain)
        got = ios_oracle.run(graph, x)
        assert np.abs(got - want).max() <= 1e-5 * max(1.0, np.abs(want).max())


def test_config_round_trip_all_models():
    for make in (ios.models.sample_network, ios.models.squeezenet_1_1, ios.models.squeezenet,
                 ios.models.randwire_small, ios.models.nasnet_mobile):
        graph = make()
        graph.sequential_schedule()
        config = json.loads(json.dumps(graph.export_config()))
        again = Graph.from_config(config)
        assert json.loads(json.dumps(again.export_config())) == config


def test_random_networks_round_trip_through_the_wire_format():
    import random_graphs
    for seed in range(0, 60, 2):
        graph, _, _ = random_graphs.random_graph(seed)
        config = json.loads(json.dumps(graph.export_config()))
        again = Graph.from_config(config)
        assert json.loads(json.dumps(again.export_config())) == config
        assert [n.name for n in again.nodes()] == [n.name for n in graph.nodes()]
        assert [tuple(n.output_shape) for n in again.nodes()] == [tuple(n.output_shape) for n in graph.nodes()]
        assert again.flops() == graph.flops() and again.kernels() == graph.kernels()


def test_model_output_shapes():
    assert tuple(ios.models.squeezenet_1_1().exit_node.output_shape) == (1000, 1, 1)
    sq = ios.models.squeezenet_1_1()
    assert [tuple(b.exit_node.output_shape) for b in sq.blocks][:4] == [(64, 55, 55), (128, 55, 55), (128, 55, 55), (128, 27, 27)]
    rw = ios.models.randwire_small()
    assert [tuple(b.exit_node.output_shape) for b in rw.blocks] == [(78, 56, 56), (78, 28, 28), (156, 14, 14),
                                                                     (312, 7, 7), (1280, 1, 1)]
    nm = ios.models.nasnet_mobile()
    assert tuple(nm.exit_node.output_shape) == (880, 1, 1)
    assert sum(len(p) for p in nm.blocks[0].parts) == len(nm.blocks[0].inner_nodes) + 1


def test_chain_and_residual_networks_of_the_zoo():
    """
    AlexNet, VGG and ResNet as the reference builds them (python/ios/models/{alexnet,vgg,resnet}.py): operator counts and
    exit shapes, and the multiply-accumulate / parameter counts of the convolutions, which are the published figures of
    these architectures (VGG-16 15.35 GMAC and 14.71 M, VGG-19 19.51 GMAC, ResNet-18 1.81 GMAC and 11.17 M, ResNet-34 3.66
    GMAC, ResNet-50 with the stride on the first 1x1 convolution 3.86 GMAC and 23.45 M; all without classifier layers).
    """
    expect = {   # name: (operators incl. placeholder, blocks, exit shape, GMAC, M parameters)
        'alexnet': (8, 1, (256, 8, 8), 0.5329, 2.469),
        'vgg_11': (15, 1, (512, 1, 1), 7.4855, 9.218),
        'vgg_13': (17, 1, (512, 1, 1), 11.1848, 9.402),
        'vgg_16': (20, 1, (512, 1, 1), 15.3466, 14.710),
        'vgg_19': (23, 1, (512, 1, 1), 19.5084, 20.019),
        'resnet18': (30, 5, (512, 7, 7), 1.8136, 11.167),
        'resnet34': (54, 5, (512, 7, 7), 3.6632, 21.268),
        'resnet50': (87, 5, (2048, 7, 7), 3.8559, 23.455),
    }
    for name, (count, blocks, exit_shape, gmac, mparam) in expect.items():
        graph = getattr(ios.models, name)()
        nodes = list(graph.nodes())
        assert [n.name for n in nodes] == [str(i) for i in range(count)], name
        assert len(graph.blocks) == blocks and tuple(graph.exit_node.output_shape) == exit_shape, name
        macs = sum(np.prod(c.output_shape) * c.fan_in for c in graph.conv_nodes())
        params = sum(np.prod(c.weight_shape) for c in graph.conv_nodes())
        assert macs / 1e9 == pytest.approx(gmac, abs=1e-4) and params / 1e6 == pytest.approx(mparam, abs=1e-3), name
        config = json.loads(json.dumps(graph.export_config()))
        assert json.loads(json.dumps(Graph.from_config(config).export_config())) == config
    r50 = {n.name: n for n in ios.models.resnet50().nodes()}
    # first residual unit: projection of the block input beside 1x1 - 3x3 - 1x1, addition of the two, in-place ReLU
    assert [r50[str(i)].type for i in range(3, 9)] == ['conv', 'conv', 'conv', 'conv', 'element', 'activation']
    assert r50['3'].act == 'relu' and r50['6'].act == 'identity' and r50['7'].op_type == 'add' and r50['8'].inplace
    assert [(v.node.name) for v in r50['7'].inputs[0]] == ['6', '3']
    # a greedy schedule runs the projection beside the first convolution of the unit
    graph = ios.models.resnet50()
    graph.greedy_schedule(8)
    assert graph.blocks[1].stages[0] == [['3'], ['4']]


def test_randwire_graph_generator_is_seeded_and_valid():
    from ios.models.randwire import watts_strogatz_edges, read_graph, write_graph
    e1 = watts_strogatz_edges(32, 4, 0.75, seed=3)
    assert e1 == watts_strogatz_edges(32, 4, 0.75, seed=3)
    assert e1 != watts_strogatz_edges(32, 4, 0.75, seed=4)
    assert len(e1) == 64 and all(0 <= u < v < 32 for u, v in e1) and len(set(e1)) == 64
    assert watts_strogatz_edges(8, 2, 0.0, seed=0) == sorted([(i, i + 1) for i in range(7)] + [(0, 7)])


def test_reference_randwire_graphs_and_the_models_built_on_them():
    """
    The edge lists the reference ships (python/ios/models/randwire_graphs/generated/, kept as fixtures under tests/golden/):
    32-node graphs with 64 edges, largest fan-in 6 / 8 / 5 / 5 over the four stages of the large model (sums of more than five
    values are what the reference adds with repeated cudnnAddTensor calls, src/ios/ios_runtime.cu:746-751), and the 320-node
    graph of the extra-large model.
    """
    from ios.models.randwire import read_graph
    graph_dir = os.path.join(GOLDEN, 'randwire_graphs')
    fan_in = []
    for fname, nodes, count in (('ws-16-4-0.75-2.txt', 16, 32), ('ws-32-4-0.75-3.txt', 32, 64), ('ws-32-4-0.75-4.txt', 32, 64),
                                ('ws-32-4-0.75-5.txt', 32, 64), ('ws-320-20-0.75-x.txt', 320, 3200)):
        n, edges = read_graph(os.path.join(graph_dir, fname))
        assert n == nodes and len(edges) == count and all(0 <= u < v < n for u, v in edges) and len(set(edges)) == count
        degree = [0] * n
        for _, v in edges:
            degree[v] += 1
        fan_in.append(max(degree))
    assert fan_in[:4] == [6, 8, 5, 5] and fan_in[4] > 8
    files = [os.path.join(graph_dir, f) for f in ('ws-16-4-0.75-2.txt', 'ws-32-4-0.75-3.txt', 'ws-32-4-0.75-4.txt', 'ws-32-4-0.75-5.txt')]
    large = ios.models.randwire_large(graph_files=files)
    assert [tuple(b.exit_node.output_shape) for b in large.blocks] == [(77, 112, 112), (154, 56, 56), (308, 28, 28), (616, 14, 14),
                                                                        (1232, 7, 7), (1280, 1, 1)]
    assert [len(b.inner_nodes) + 1 for b in large.blocks[1:5]] == [17, 33, 33, 33]      # nodes + the summing exit
    assert max(len(n.nodes[0].inputs[0]) for b in large.blocks[1:5] for n in b.inner_nodes) == 8
    seeded = ios.models.randwire_large()                                                   # generated graphs, same parameters
    assert [tuple(b.exit_node.output_shape) for b in seeded.blocks] == [tuple(b.exit_node.output_shape) for b in large.blocks]
    xlarge = ios.models.randwire_xlarge(graph_file=os.path.join(graph_dir, 'ws-320-20-0.75-x.txt'))
    generated = ios.models.randwire_xlarge()
    assert len(generated.blocks[1].inner_nodes) == 320 and generated.blocks[1].exit_node.output_shape == xlarge.blocks[1].exit_node.output_shape
    assert len(xlarge.blocks) == 3 and len(xlarge.blocks[1].inner_nodes) == 320 and tuple(xlarge.exit_node.output_shape) == (1280, 1, 1)


def test_randwire_edge_file_format(tmp_path):
    from ios.models.randwire import watts_strogatz_edges, read_graph, write_graph
    edges = watts_strogatz_edges(16, 4, 0.75, seed=2)
    path = tmp_path / 'ws.txt'
    write_graph(path, 16, edges)
    assert read_graph(path) == (16, edges)


def test_sequential_and_greedy_schedules_cover_all_operators():
    graph = ios.models.inception_v3()
    for schedule in (graph.sequential_schedule, lambda: graph.greedy_schedule(4)):
        schedule()
        for block in graph.blocks:
            names = [n for stage in block.stages for group in stage for n in group]
            assert sorted(names) == sorted(n.name for n in block.inner_nodes + [block.exit_node])
            assert all(len(stage) <= 4 or schedule == graph.sequential_schedule for stage in block.stages)
    graph.greedy_schedule(10)
    # inception_a block: the four branch heads are ready at once
    assert graph.blocks[1].stages[0] == [['8'], ['9'], ['11'], ['14']]


def test_seeded_he_normal_init():
    g1 = ios.models.sample_network(init_seed=0, init_scheme='he_normal')
    g2 = ios.models.sample_network(init_seed=0, init_scheme='he_normal')
    c1, c2 = g1.conv_nodes()[0], g2.conv_nodes()[0]
    np.testing.assert_array_equal(c1.weight, c2.weight)
    assert c1.weight.dtype == np.float32 and c1.weight.shape == (375, 375, 3, 3)
    assert np.all(c1.bias == 0)
    assert c1.weight.std() == pytest.approx(np.sqrt(2.0 / (375 * 9)), rel=0.02)


def test_value_and_uses():
    ios.reset_name()
    v = ios.placeholder((8, 4, 4))
    block = ios.Block(v.node)
    a = ios.conv2d(block, [[v]], 8)
    b = ios.identity(block, [[a, v]], is_exit=True)
    assert a.node.uses == [(b.node, 0, 0)]
    assert v.node.uses == [(a.node, 0, 0), (b.node, 0, 1)]
    assert Value(a.node, 0, 8) == a and a.length == 8
    assert b.node.input_readable_str() == '(1+0)'


def test_draw_writes_graphviz_source_without_pydot(tmp_path):
    from ios.visualizer import to_dot
    graph = ios.models.sample_network()
    graph.blocks[0].stages = [[['1'], ['2']], [['4'], ['3']], [['5']]]
    source = to_dot(graph, label='demo')
    assert source.startswith('digraph') and source.count('->') == 7 and 'subgraph cluster_0' in source
    for name, stage in (('1', 0), ('2', 0), ('4', 1), ('3', 1), ('5', 2)):
        assert f'{name} @ stage {stage}' in source
    assert source.count('fillcolor=lightblue') == 2      # the two operators of the first stage share a colour
    target = ios.draw(graph, str(tmp_path / 'demo.gv'), label='demo')
    assert open(target).read() == source
    # slices and summed values are marked on their edges; every operator of a large network is drawn once
    nasnet = ios.models.nasnet_mobile()
    nasnet.greedy_schedule(8)
    text = to_dot(nasnet)
    assert text.count('arrowhead=odot') > 50 and sum(1 for line in text.splitlines() if 'fillcolor=' in line and '->' not in line) == \
           1 + sum(len(b.inner_nodes) + 1 for b in nasnet.blocks)
    merged = Graph.from_config(json.load(open(os.path.join(GOLDEN, 'inception_v3_dp_parallel_merge.json'))))
    assert '[' in to_dot(merged) and ':' in to_dot(merged)      # channel slices of merged convolutions


def test_unknown_node_type_raises():
    with pytest.raises(ValueError):
        ios.ir.Node.from_config({'type': 'softmax', 'name': 'x', 'hint_name': 'x', 'inputs': [], 'output_shape': None}, {})
