"""
GPU parity: the HIP runtime, called through its C ABI, against the CPU oracle on the same seeded inputs.
Tolerance for fp32: |got - want| <= 1e-4 + 1e-3 * |want| (rel 1e-3 / abs 1e-4), element by element, everywhere
except NASNet under the He-normal initialisation its configuration names: without normalisation its activations
reach 1e5, where one fp32 rounding is 8e-3, so that case is held to the same formula with the absolute part scaled
by the tensor's largest magnitude and reports how many elements miss the unscaled formula and by how many ulps.
Whole networks run with seeded non-zero biases.  With the kernel configuration pinned, schedule and executor
changes must not change results at all.
"""
import os

import numpy as np
import pytest

import ios
from ios.contrib import ios_runtime as rt
from ios.ir import Graph, Value
from oracle import ios_oracle

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-3, 1e-4


def assert_close(got, want, what='', scaled=False):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    scale = max(1.0, float(np.abs(want).max())) if (scaled and want.size) else 1.0
    bound = ATOL * scale + RTOL * np.abs(want.astype(np.float64))
    bad = err > bound
    assert not bad.any(), (f'{what}: {bad.sum()} of {bad.size} elements out of tolerance, max abs err '
                           f'{err.max():.3e} at {np.unravel_index(err.argmax(), err.shape)}, '
                           f'want there {want.flat[err.argmax()]:.6f} got {got.flat[err.argmax()]:.6f}')


@pytest.fixture(autouse=True)
def default_options():
    rt.set_option('conv_variant', -1)
    rt.set_option('conv_split_k', 0)
    rt.set_option('executor', 'streams')
    rt.set_option('autotune', 0)            # closed-form kernel configurations keep the suite short and repeatable
    rt.set_option('split_k_reduce', 'xcd')   # the library's default: K slices of a tile meet inside one XCD
    rt.set_option('precision', 'fp32')
    rt.set_option('arena_reuse', 1)
    rt.set_option('thin_conv_min_pixels', 1 << 18)
    yield
    rt.set_option('arena_reuse', 1)
    rt.set_option('thin_conv_min_pixels', 1 << 18)
    rt.set_option('precision', 'fp32')
    rt.set_option('autotune', 0)
    rt.set_option('conv_variant', -1)
    rt.set_option('conv_split_k', 0)
    rt.set_option('executor', 'streams')
    rt.set_option('split_k_reduce', 'xcd')


def single_op_graph(in_shape, build):
    ios.reset_name()
    v = ios.placeholder(in_shape)
    block = ios.Block(v.node)
    build(block, v)
    graph = Graph('t', v.node, [block])
    graph.init_weights(seed=7, scheme='he_normal')
    for conv in graph.conv_nodes():   # non-zero bias so that a dropped bias fails
        conv.bias = np.random.default_rng(int(conv.name) + 100).standard_normal(conv.bias.shape).astype(np.float32) * 0.5
    graph.sequential_schedule()
    return graph


def run_both(graph, batch, seed=1):
    x = np.random.default_rng(seed).standard_normal((batch, *graph.enter_node.output_shape)).astype(np.float32)
    got = rt.graph_inference(graph, batch, x)
    want = ios_oracle.run(graph, x)
    assert got.shape == want.shape
    return got, want


CONVS = [
    # in_shape, out_channels, kernel, stride, padding, groups, act, batch
    ((16, 9, 9), 24, (3, 3), (1, 1), (1, 1), 1, 'relu', 1),
    ((3, 31, 31), 32, (3, 3), (2, 2), (0, 0), 1, 'relu', 2),
    ((48, 17, 17), 64, (5, 5), (1, 1), (2, 2), 1, 'relu', 1),
    ((40, 17, 17), 48, (1, 7), (1, 1), (0, 3), 1, 'relu', 1),
    ((40, 17, 17), 48, (7, 1), (1, 1), (3, 0), 1, 'identity', 3),
    ((192, 8, 8), 100, (1, 1), (1, 1), (0, 0), 1, 'tanh', 1),
    ((70, 12, 12), 33, (1, 1), (2, 2), (0, 0), 1, 'sigmoid', 2),
    ((375, 15, 15), 75, (3, 3), (1, 1), (1, 1), 1, 'relu', 1),       # odd channel counts (sample net)
    ((32, 14, 14), 32, (3, 3), (1, 1), (1, 1), 32, 'identity', 2),   # depthwise 3x3
    ((24, 15, 15), 24, (5, 5), (2, 2), (2, 2), 24, 'identity', 1),   # depthwise 5x5 strided
    ((16, 13, 13), 16, (7, 7), (2, 2), (3, 3), 16, 'relu', 1),       # depthwise 7x7
    ((32, 10, 10), 48, (3, 3), (1, 1), (1, 1), 4, 'relu', 2),        # grouped, matrix path per group
    ((12, 10, 10), 12, (3, 3), (1, 1), (1, 1), 6, 'relu', 1),        # thin groups, direct path
    ((8, 7, 7), 10, (3, 3), (1, 1), (2, 2), 1, 'identity', 1),       # padding larger than "same"
]


@pytest.mark.parametrize('case', CONVS)
def test_conv_matches_oracle(case):
    in_shape, oc, k, s, p, g, act, batch = case
    graph = single_op_graph(in_shape, lambda b, v: ios.conv2d(b, [[v]], oc, k, s, p, g, act, is_exit=True))
    got, want = run_both(graph, batch)
    assert_close(got, want, f'conv {case}')


def test_committed_operator_vectors():
    """The fixed inputs, weights and brute-force outputs of tests/golden/operator_vectors.npz through the C ABI."""
    import os
    import sys
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')
    sys.path.insert(0, golden)
    import make_operator_vectors as spec
    data = np.load(os.path.join(golden, 'operator_vectors.npz'))
    for name, shape, oc, kernel, stride, padding, groups, act in spec.CONVS:
        graph = single_op_graph(shape[1:], lambda b, v: ios.conv2d(b, [[v]], oc, kernel, stride, padding, groups, act, is_exit=True))
        conv = list(graph.conv_nodes())[0]
        conv.weight, conv.bias = data[f'{name}.w'], data[f'{name}.b']
        got = rt.graph_inference(graph, shape[0], data[f'{name}.x'])
        assert_close(got, data[f'{name}.y'], name)
    for name, shape, pool_type, kernel, stride, padding in spec.POOLS:
        graph = single_op_graph(shape[1:], lambda b, v: ios.pool2d(b, [[v]], pool_type, kernel, stride, padding, is_exit=True))
        got = rt.graph_inference(graph, shape[0], data[f'{name}.x'])
        assert_close(got, data[f'{name}.y'], name)


# every fp32 kernel configuration the library was built with (host-only query; the bfloat16 ones have their own test)
FP32_VARIANTS = [name for name in rt.conv_variant_names() if not name.startswith(('wb_', 'wh_'))]


@pytest.mark.parametrize('variant_name', FP32_VARIANTS)
@pytest.mark.parametrize('split_k', [1, 3])
def test_every_conv_kernel_variant(variant_name, split_k):
    variant = rt.device_info()['conv_variants'].index(variant_name)
    rt.set_option('conv_variant', variant)
    rt.set_option('conv_split_k', split_k)
    for in_shape, oc, k, s, p, batch in [((72, 19, 19), 88, (3, 3), (1, 1), (1, 1), 2),
                                          ((200, 8, 8), 136, (1, 1), (1, 1), (0, 0), 1),
                                          ((20, 37, 37), 24, (5, 5), (2, 2), (2, 2), 1)]:
        graph = single_op_graph(in_shape, lambda b, v: ios.conv2d(b, [[v]], oc, k, s, p, 1, 'relu', is_exit=True))
        got, want = run_both(graph, batch)
        assert_close(got, want, f'variant {variant} split {split_k} conv {in_shape}->{oc} {k}')
        got2, _ = run_both(graph, batch)
        np.testing.assert_array_equal(got, got2)      # split-K reduction order is fixed


def residual_unit_graph(in_shape, oc, k, s, p, act, relu, conv_first=True, skip_slice=False):
    """skip = conv(x) (a channel slice of a wider convolution when `skip_slice`); y = conv(x); exit = [relu](y + skip)."""
    ios.reset_name()
    v = ios.placeholder(in_shape)
    unit = ios.Block(v.node)
    extra = 3 if skip_slice else 0
    wide = ios.conv2d(unit, [[v]], oc + extra, k, s, p, 1, 'tanh')
    skip = Value(wide.node, extra, oc + extra)
    y = ios.conv2d(unit, [[v]], oc, k, s, p, 1, act)
    pair = [y, skip] if conv_first else [skip, y]
    if relu:
        e = ios.addition(unit, [pair])
        ios.activation(unit, [[e]], 'relu', True, is_exit=True)
    else:
        ios.addition(unit, [pair], is_exit=True)
    graph = Graph('residual', v.node, [unit])
    graph.init_weights(0, 'he_normal_bias')
    graph.sequential_schedule()
    return graph


@pytest.mark.parametrize('variant_name', FP32_VARIANTS)
@pytest.mark.parametrize('split_k', [1, 3])
def test_residual_epilogue_of_every_conv_kernel_variant(variant_name, split_k):
    """out = [relu](act(conv + bias) + skip) in the convolution's epilogue (both split-K reductions included) equals the
    oracle's three operators; the plan holds no launch for the addition."""
    variant = rt.device_info()['conv_variants'].index(variant_name)
    rt.set_option('conv_variant', variant)
    rt.set_option('conv_split_k', split_k)
    cases = [((72, 19, 19), 88, (3, 3), (1, 1), (1, 1), 'identity', True, True, False, 2),
             ((200, 8, 8), 136, (1, 1), (1, 1), (0, 0), 'relu', False, False, True, 1),
             ((20, 37, 37), 24, (5, 5), (2, 2), (2, 2), 'identity', True, False, True, 3)]
    for in_shape, oc, k, s, p, act, relu, conv_first, skip_slice, batch in cases:
        graph = residual_unit_graph(in_shape, oc, k, s, p, act, relu, conv_first, skip_slice)
        ops = rt.plan_describe(graph, batch)
        assert [op['kind'] for op in ops] == ['conv_mfma', 'conv_mfma'] and ops[1]['residual'] and ops[1]['post_relu'] == int(relu)
        x = np.random.default_rng(3).standard_normal((batch, *in_shape)).astype(np.float32)
        want = ios_oracle.run(graph, x)
        for reduce in ('xcd', 'inline', 'kernel'):       # (a residual convolution under 'xcd' takes the device-wide form)
            rt.set_option('split_k_reduce', reduce)
            got = rt.graph_inference(graph, batch, x)
            assert_close(got, want, f'variant {variant_name} split {split_k} ({reduce}) residual unit {in_shape}->{oc} {k}')


def test_residual_unit_under_every_executor_and_without_the_matrix_path():
    graph = residual_unit_graph((24, 15, 15), 40, (3, 3), (1, 1), (1, 1), 'identity', True)
    x = np.random.default_rng(2).standard_normal((3, 24, 15, 15)).astype(np.float32)
    want = ios_oracle.run(graph, x)
    first = None
    for executor in ('streams', 'graph', 'fused', 'fused_graph'):
        rt.set_option('executor', executor)
        with rt.Session(graph, 3) as session:
            session.load_weights()
            session.set_input(x)
            for _ in range(2):
                session.run()
            got = session.output()
            with pytest.raises(RuntimeError, match='no materialised output'):      # the convolution wrote the ReLU's tensor
                session.tensor([n for n in graph.nodes() if n.type == 'conv'][1])
        assert_close(got, want, f'residual unit, {executor}')
        first = got if first is None else first
        np.testing.assert_array_equal(got, first)
    rt.set_option('executor', 'streams')
    # a depth-wise convolution in the same place keeps its own launch and the addition follows
    ios.reset_name()
    v = ios.placeholder((24, 15, 15))
    block = ios.Block(v.node)
    skip = ios.conv2d(block, [[v]], 24, (1, 1), act='identity')
    y = ios.conv2d(block, [[v]], 24, (3, 3), (1, 1), (1, 1), 24, 'identity')
    e = ios.addition(block, [[y, skip]])
    ios.relu(block, [[e]], is_exit=True)
    graph = Graph('residual_depthwise', v.node, [block])
    graph.init_weights(0, 'he_normal_bias')
    graph.sequential_schedule()
    assert [op['kind'] for op in rt.plan_describe(graph, 3)] == ['conv_mfma', 'conv_depthwise', 'nary']
    assert_close(rt.graph_inference(graph, 3, x), ios_oracle.run(graph, x), 'depth-wise convolution, addition, ReLU')


@pytest.mark.parametrize('variant_name', ['ws_m32n32_w1_t16_c4', 'ws_m32n64_w1_t16_c4', 'ws_m32n32_w2_t16_c4', 'ws_m32n16_w4_t16_c4'])
def test_first_layer_configurations_on_three_and_five_channel_inputs(variant_name):
    """Channel padding 4: K = taps x 4 (3 channels) or taps x 8 (5 channels), strided, with and without padding."""
    names = rt.device_info()['conv_variants']
    rt.set_option('conv_variant', names.index(variant_name))
    rt.set_option('conv_split_k', 1)
    for in_shape, oc, k, s, p, batch in [((3, 41, 41), 32, (3, 3), (2, 2), (0, 0), 2), ((3, 23, 29), 39, (3, 3), (2, 2), (1, 1), 1),
                                          ((5, 17, 17), 20, (5, 5), (1, 1), (2, 2), 3), ((1, 19, 19), 8, (7, 7), (2, 2), (3, 3), 1)]:
        graph = single_op_graph(in_shape, lambda b, v: ios.conv2d(b, [[v]], oc, k, s, p, 1, 'relu', is_exit=True))
        got, want = run_both(graph, batch)
        assert_close(got, want, f'{variant_name} conv {in_shape}->{oc} {k}')


@pytest.mark.parametrize('variant_name', ['m64n64k32_w2x2x1_t32', 'm32n32k64_w1x1x4_t32', 'm64n16k64_w4x1x1_t16',
                                          'm32n16k64_w2x1x2_t16', 'm128n64k16_w2x2x1_t32', 'ws_m32n16_w8_t16',
                                          'wq_m16n16_w16_t16', 'wq_m32n32_w16_t16', 'ws_m32n32_w16_t32'])
def test_split_k_reduction_inside_the_kernel_equals_the_reduction_kernel(variant_name):
    """All three forms (second kernel, last block with the slices anywhere on the device, last block with the slices of a tile
    on one XCD) add the same partial tiles in slice order, so they must agree bit for bit, launch after launch."""
    info = rt.device_info()
    assert info['xcd_placement_probe'], 'blocks with equal index % 8 did not share an XCC: the XCD-local form is not exercised'
    names = info['conv_variants']
    rt.set_option('conv_variant', names.index(variant_name))
    for in_shape, oc, k, p, batch, split in [((200, 8, 8), 136, (1, 1), (0, 0), 1, 6), ((72, 19, 19), 88, (3, 3), (1, 1), 2, 3),
                                             ((96, 17, 17), 40, (1, 7), (0, 3), 1, 4)]:
        rt.set_option('conv_split_k', split)
        graph = single_op_graph(in_shape, lambda b, v: ios.conv2d(b, [[v]], oc, k, (1, 1), p, 1, 'relu', is_exit=True))
        x = np.random.default_rng(5).standard_normal((batch, *in_shape)).astype(np.float32)
        want = ios_oracle.run(graph, x)
        results = {}
        for form in ('kernel', 'inline', 'xcd'):
            rt.set_option('split_k_reduce', form)
            with rt.Session(graph, batch) as session:
                session.load_weights()
                session.set_input(x)
                outs = []
                for _ in range(4):          # the tickets must be back at zero after every launch
                    session.run()
                    outs.append(session.output())
                for out in outs[1:]:
                    np.testing.assert_array_equal(outs[0], out)
                results[form] = outs[0]
        assert_close(results['inline'], want, f'{variant_name} split {split} {in_shape}')
        np.testing.assert_array_equal(results['inline'], results['kernel'])
        np.testing.assert_array_equal(results['xcd'], results['kernel'])


def test_bfloat16_split_kernels_are_as_accurate_as_the_fp32_matrix_instructions():
    """The x3_* configurations compute fp32 products as six bfloat16 products of exactly split operands: against a float64
    reference their error must be of the size of the fp32 kernels' own (not of bfloat16's), on a long K."""
    import torch
    names = rt.device_info()['conv_variants']
    in_shape, oc, batch = (256, 17, 17), 96, 2
    graph = single_op_graph(in_shape, lambda b, v: ios.conv2d(b, [[v]], oc, (3, 3), (1, 1), (1, 1), 1, 'identity', is_exit=True))
    x = np.random.default_rng(11).standard_normal((batch, *in_shape)).astype(np.float32)
    conv = list(graph.conv_nodes())[0]
    want = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(conv.weight).double(),
                                      torch.from_numpy(conv.bias).double(), padding=1).numpy()
    scale = np.abs(want).max()
    errors = {}
    for name in ('wq_m32n16_w8_t16', 'm64n64k32_w2x2x1_t32', 'x3_m64n128_w2x2', 'x3_m64n64_w1x1', 'x3_m128n64_w4x1'):
        rt.set_option('conv_variant', names.index(name))
        got = rt.graph_inference(graph, batch, x)
        errors[name] = np.abs(got - want).max() / scale
    fp32 = max(errors['wq_m32n16_w8_t16'], errors['m64n64k32_w2x2x1_t32'])
    assert fp32 < 2e-6, errors                                   # K = 2304 fp32 accumulation
    for name, err in errors.items():
        if name.startswith('x3_'):
            assert err < 2.0 * fp32 + 1e-7, errors               # bfloat16 operands alone would give ~4e-3


def test_split_k_is_repeatable_in_a_session():
    rt.set_option('conv_split_k', 4)
    graph = single_op_graph((64, 12, 12), lambda b, v: ios.conv2d(b, [[v]], 40, (3, 3), (1, 1), (1, 1), 1, 'relu', is_exit=True))
    x = np.random.default_rng(3).standard_normal((2, 64, 12, 12)).astype(np.float32)
    want = ios_oracle.run(graph, x)
    with rt.Session(graph, 2) as session:
        session.load_weights()
        session.set_input(x)
        for _ in range(3):
            session.run()
            assert_close(session.output(), want, 'repeated split-K run')


POOLS = [
    ((24, 35, 35), 'max', (3, 3), (2, 2), (0, 0), 1),
    ((24, 17, 17), 'avg', (3, 3), (1, 1), (1, 1), 2),
    ((10, 14, 14), 'max', (3, 3), (2, 2), (1, 1), 1),
    ((10, 15, 15), 'avg', (3, 3), (2, 2), (1, 1), 1),
    ((6, 8, 8), 'max', (2, 2), (2, 2), (0, 0), 3),
    ((40, 8, 8), 'global_avg', (1, 1), (1, 1), (0, 0), 2),
    ((9, 13, 13), 'global_max', (1, 1), (1, 1), (0, 0), 1),
    # large enough for the 3 x 3 kernel to give every thread a strip of 8, 8, 8, 4 and 2 output rows
    ((64, 147, 147), 'avg', (3, 3), (1, 1), (1, 1), 8),
    ((64, 147, 147), 'max', (3, 3), (1, 1), (1, 1), 8),
    ((128, 149, 149), 'max', (3, 3), (2, 2), (0, 0), 16),
    ((96, 75, 75), 'avg', (3, 3), (2, 2), (1, 1), 32),
    ((64, 75, 75), 'max', (3, 3), (1, 2), (1, 0), 8),
]


COMMUTED = [
    # in_shape, out_channels, act, pool kernel / stride / padding, batch, executor: average pools that keep the map size in
    # front of a 1 x 1 convolution to no more channels (every pool body: one column, four columns, generic window)
    ((48, 17, 17), 24, 'relu', (3, 3), (1, 1), (1, 1), 3, 'streams'),
    ((64, 35, 35), 64, 'identity', (3, 3), (1, 1), (1, 1), 16, 'fused'),        # four output columns per thread
    ((20, 9, 11), 7, 'tanh', (5, 5), (1, 1), (2, 2), 2, 'streams'),              # generic window, odd channel count
    ((96, 8, 8), 32, 'sigmoid', (3, 3), (1, 1), (1, 1), 1, 'fused_graph'),
]


@pytest.mark.parametrize('case', COMMUTED, ids=[f'{c[0][0]}x{c[0][1]}x{c[0][2]}-{c[1]}-{c[2]}' for c in COMMUTED])
def test_average_pool_exchanged_with_its_pointwise_convolution_matches_oracle(case):
    """
    y = act(W * avgpool(x) + b) computed as act(avgpool(W * x) + b): the border elements, where the window counts padding
    (the divisor stays KH * KW, reference src/ios/ios_runtime.cu:542-550), bias and activation included.  A second reader of
    the pool, a max pool, a pool that changes the map size and a 3 x 3 convolution keep the reference's order.
    """
    in_shape, oc, act, kernel, stride, padding, batch, executor = case

    def build(b, v):
        pooled = ios.pool2d(b, [[v]], 'avg', kernel, stride, padding)
        ios.conv2d(b, [[pooled]], oc, (1, 1), (1, 1), (0, 0), 1, act, is_exit=True)

    graph = single_op_graph(in_shape, build)
    rt.set_option('executor', executor)
    try:
        ops = rt.plan_describe(graph, batch)
        assert [bool(op.get('linear')) for op in ops] == [True, False] and ops[1]['kind'] == 'pool' and 'adds_bias_of' in ops[1]
        got, want = run_both(graph, batch)
        assert_close(got, want, f'exchanged pool {case}')
        # border rows and columns on their own: a wrong divisor or a bias added before the pool shows there first
        for border in (got[:, :, 0, :] - want[:, :, 0, :], got[:, :, :, -1] - want[:, :, :, -1]):
            assert np.abs(border).max() <= 1e-4 + 1e-3 * np.abs(want).max()
        rt.set_option('commute_pool_conv', 0)
        plain = rt.graph_inference(graph, batch, np.random.default_rng(1).standard_normal((batch, *in_shape)).astype(np.float32))
        assert_close(plain, want, f'reference order {case}')
        assert not any(op.get('linear') for op in rt.plan_describe(graph, batch))
    finally:
        rt.set_option('commute_pool_conv', 1)
        rt.set_option('executor', 'streams')


def test_pools_that_must_keep_their_place():
    def two_readers(b, v):
        pooled = ios.pool2d(b, [[v]], 'avg', (3, 3), (1, 1), (1, 1))
        c = ios.conv2d(b, [[pooled]], 16, (1, 1), (1, 1), (0, 0), 1, 'relu')
        ios.identity(b, [[c], [pooled]], is_exit=True)

    def max_pool(b, v):
        ios.conv2d(b, [[ios.pool2d(b, [[v]], 'max', (3, 3), (1, 1), (1, 1))]], 16, (1, 1), (1, 1), (0, 0), 1, 'relu', is_exit=True)

    def shrinking(b, v):
        ios.conv2d(b, [[ios.pool2d(b, [[v]], 'avg', (3, 3), (2, 2), (1, 1))]], 16, (1, 1), (1, 1), (0, 0), 1, 'relu', is_exit=True)

    def wide_window(b, v):
        ios.conv2d(b, [[ios.pool2d(b, [[v]], 'avg', (3, 3), (1, 1), (1, 1))]], 16, (3, 3), (1, 1), (1, 1), 1, 'relu', is_exit=True)

    def more_channels(b, v):
        ios.conv2d(b, [[ios.pool2d(b, [[v]], 'avg', (3, 3), (1, 1), (1, 1))]], 64, (1, 1), (1, 1), (0, 0), 1, 'relu', is_exit=True)

    for build in (two_readers, max_pool, shrinking, wide_window, more_channels):
        graph = single_op_graph((24, 14, 14), build)
        assert not any(op.get('linear') for op in rt.plan_describe(graph, 2)), build.__name__
        got, want = run_both(graph, 2)
        assert_close(got, want, build.__name__)


@pytest.mark.parametrize('case', POOLS)
def test_pool_matches_oracle(case):
    in_shape, kind, k, s, p, batch = case
    graph = single_op_graph(in_shape, lambda b, v: ios.pool2d(b, [[v]], kind, k, s, p, is_exit=True))
    x = np.random.default_rng(2).standard_normal((batch, *in_shape)).astype(np.float32) - 2.0   # mostly negative
    got = rt.graph_inference(graph, batch, x)
    want = ios_oracle.run(graph, x)
    assert_close(got, want, f'pool {case}')


THIN_CONVS = [
    # 3 x 3 convolutions of 3-channel images on the output-bound direct kernel: in_shape, out_channels, stride, padding, act, batch
    ((3, 31, 31), 32, 2, 0, 'relu', 2),
    ((3, 30, 33), 40, 2, 1, 'relu', 3),         # output channels that do not fill the second block of 32, padding
    ((3, 19, 17), 70, 1, 1, 'identity', 1),
    ((3, 64, 64), 24, 1, 0, 'tanh', 5),         # fewer than 32 output channels
    ((3, 299, 299), 32, 2, 0, 'relu', 4),       # Inception-v3's first layer, above the default size threshold
]


@pytest.mark.parametrize('case', THIN_CONVS)
def test_first_layer_kernel_for_three_channel_images_matches_oracle(case):
    in_shape, oc, stride, pad, act, batch = case
    def build(b, v):
        a = ios.conv2d(b, [[v]], oc, (3, 3), (stride, stride), (pad, pad), act=act)
        c = ios.conv2d(b, [[a]], 8, (1, 1))
        ios.identity(b, [[c], [a]], is_exit=True)       # the convolution stores into a channel window
    graph = single_op_graph(in_shape, build)
    rt.set_option('thin_conv_min_pixels', 0 if in_shape[1] < 100 else 1 << 16)
    first = rt.plan_describe(graph, batch)[0]
    assert first['kind'] == 'conv_direct' and first['thin'] is True
    x = np.random.default_rng(6).standard_normal((batch, *in_shape)).astype(np.float32)
    want = ios_oracle.run(graph, x)
    outs = {}
    for executor in ('streams', 'fused', 'fused_graph'):
        rt.set_option('executor', executor)
        outs[executor] = rt.graph_inference(graph, batch, x)
        assert_close(outs[executor], want, f'thin conv {case} {executor}')
    rt.set_option('thin_conv_min_pixels', -1)
    assert rt.plan_describe(graph, batch)[0]['kind'] == 'conv_mfma'
    assert_close(rt.graph_inference(graph, batch, x), want, f'matrix path {case}')


def test_first_layer_kernel_stays_out_of_stages_with_several_groups():
    def build(b, v):
        a = ios.conv2d(b, [[v]], 32, (3, 3), (2, 2))
        c = ios.conv2d(b, [[v]], 16, (3, 3), (2, 2))
        ios.identity(b, [[a], [c]], is_exit=True)
    graph = single_op_graph((3, 40, 40), build)
    rt.set_option('thin_conv_min_pixels', 0)
    assert [op['kind'] for op in rt.plan_describe(graph, 2)] == ['conv_direct', 'conv_direct']
    names = [n.name for n in graph.blocks[0].inner_nodes]
    graph.blocks[0].stages = [[[names[0]], [names[1]]], [[graph.blocks[0].exit_node.name]]]
    assert [op['kind'] for op in rt.plan_describe(graph, 2)] == ['conv_mfma', 'conv_mfma']
    x = np.random.default_rng(8).standard_normal((2, 3, 40, 40)).astype(np.float32)
    rt.set_option('executor', 'fused')
    assert_close(rt.graph_inference(graph, 2, x), ios_oracle.run(graph, x), 'parallel first layers')


LARGE_POOLS = [
    # tensors large enough for the form with four output columns per thread (16-byte loads at any alignment, reads past
    # the end of a row that must be discarded): in_shape, type, stride, padding, batch
    ((128, 35, 35), 'avg', 1, 1, 16),       # OW = 35: the last thread of a row holds three columns
    ((128, 35, 35), 'max', 1, 1, 16),
    ((96, 71, 71), 'max', 2, 0, 8),         # Inception-v3 reduction pools: odd width, no padding
    ((176, 56, 56), 'avg', 2, 1, 16),       # NASNet: stride 2 with padding, even width
    ((176, 56, 56), 'max', 2, 1, 16),
    ((640, 9, 10), 'avg', 1, 1, 32),        # rows shorter than three threads' worth, width != height
    ((512, 17, 17), 'max', 1, 0, 16),       # no padding: OW = 15
]


@pytest.mark.parametrize('case', LARGE_POOLS)
def test_large_pool_with_four_columns_per_thread_matches_oracle(case):
    in_shape, kind, stride, pad, batch = case
    def build(b, v):
        # the pool reads a channel window of the input and writes into a channel window of the concatenation
        mid = Value(v.node, 3, in_shape[0] - 2)
        a = ios.pool2d(b, [[mid]], kind, (3, 3), (stride, stride), (pad, pad))
        c = ios.pool2d(b, [[Value(v.node, 0, 4)]], 'max' if kind == 'avg' else 'avg', (3, 3), (stride, stride), (pad, pad))
        ios.identity(b, [[c], [a]], is_exit=True)
    graph = single_op_graph(in_shape, build)
    x = np.random.default_rng(5).standard_normal((batch, *in_shape)).astype(np.float32) - 2.0
    want = ios_oracle.run(graph, x)
    for executor in ('streams', 'fused'):
        rt.set_option('executor', executor)
        got = rt.graph_inference(graph, batch, x)
        assert_close(got, want, f'large pool {case} {executor}')


def test_input_algebra_sum_concat_slice_activation_element():
    def build(b, v):
        a = ios.conv2d(b, [[v]], 12, (1, 1), act='identity')
        c = ios.conv2d(b, [[v]], 12, (3, 3), padding=(1, 1), act='identity')
        s = ios.identity(b, [[a, c, a]])                                   # three-way sum
        cat = ios.identity(b, [[a], [Value(c.node, 2, 8)], [a, c]])        # concat of value, slice, sum
        r = ios.relu(b, [[cat]])
        t = ios.activation(b, [[s], [Value(r.node, 0, 6)]], 'tanh', False)
        m = ios.multiply(b, [[a, c]])
        e = ios.addition(b, [[m, s]])
        p = ios.pool2d(b, [[e, a]], 'avg', (3, 3), (1, 1), (1, 1))          # pool over a summed input
        q = ios.conv2d(b, [[t], [p]], 10, (3, 3), padding=(1, 1))           # conv over a concatenated input
        ios.identity(b, [[q], [Value(r.node, 3, 30)], [Value(t.node, 1, 18)]], is_exit=True)
    graph = single_op_graph((5, 11, 11), build)
    for batch in (1, 3):
        x = np.random.default_rng(4).standard_normal((batch, 5, 11, 11)).astype(np.float32)
        want = ios_oracle.run(graph, x, keep_all=True)
        rt.set_option('arena_reuse', 0)      # every operator's output survives the pass
        with rt.Session(graph, batch) as session:
            session.load_weights()
            session.set_input(x)
            session.run()
            for node in list(graph.nodes())[1:]:
                assert_close(session.tensor(node), want[node.name], f'node {node.name} ({node.type}) batch {batch}')
        rt.set_option('arena_reuse', 1)
        with rt.Session(graph, batch) as session:
            session.load_weights()
            session.set_input(x)
            for _ in range(2):      # the second pass finds the input where the first one left it
                session.run()
            assert_close(session.output(), want[graph.exit_node.name], f'shared arena, batch {batch}')
            unreadable = 0
            for node in list(graph.nodes())[1:]:
                try:
                    assert_close(session.tensor(node), want[node.name], f'node {node.name} ({node.type}) batch {batch}, shared arena')
                except RuntimeError as error:      # refused, not garbage: the node's memory was given to a later operator
                    assert 'does not survive' in str(error)
                    unreadable += 1
            assert unreadable > 0


def test_fused_stage_launch_covers_every_operator_kind():
    # one stage whose groups hold every kind of device operation, run as fused launches and on streams
    def build(b, v):
        a = ios.conv2d(b, [[v]], 40, (3, 3), padding=(1, 1))                       # matrix path
        c = ios.conv2d(b, [[v]], 16, (3, 3), padding=(1, 1), groups=16)            # depth-wise
        d = ios.conv2d(b, [[v]], 16, (3, 3), padding=(1, 1), groups=8)             # thin groups: direct path
        e = ios.pool2d(b, [[v]], 'avg', (3, 3), (1, 1), (1, 1))
        f = ios.pool2d(b, [[v]], 'global_avg')
        s = ios.relu(b, [[v, v]])
        u = ios.activation(b, [[Value(v.node, 2, 9)]], 'tanh', False)
        a2 = ios.conv2d(b, [[a]], 24, (1, 1))
        s2 = ios.relu_sep_conv(b, [[s]], 12, (3, 3), (1, 1), (1, 1))
        ios.identity(b, [[a2], [c], [d], [e], [s2], [u]], is_exit=True)
        return f
    graph = single_op_graph((16, 14, 14), build)
    names = [n.name for n in graph.blocks[0].inner_nodes]
    # groups: conv chain, the others one per group
    graph.blocks[0].stages = [[[names[0], names[7]], [names[1]], [names[2]], [names[3]], [names[4]], [names[5], names[8]], [names[6]]],
                              [[graph.blocks[0].exit_node.name]]]
    for split in (0, 3):
        rt.set_option('conv_split_k', split)
        names = rt.device_info()['conv_variants']
        for variant in (-1, names.index('wq_m32n32_w4_t16'), names.index('wq_m32n16_w8_t16'), names.index('ws_m32n16_w16_t16')):
            rt.set_option('conv_variant', variant)
            for batch in (1, 2):
                x = np.random.default_rng(5).standard_normal((batch, 16, 14, 14)).astype(np.float32)
                want = ios_oracle.run(graph, x)
                outs = {}
                for executor in ('streams', 'fused', 'fused_graph'):
                    rt.set_option('executor', executor)
                    outs[executor] = rt.graph_inference(graph, batch, x)
                    assert_close(outs[executor], want, f'{executor} split {split} variant {variant} batch {batch}')
                np.testing.assert_array_equal(outs['fused'], outs['streams'])
                np.testing.assert_array_equal(outs['fused_graph'], outs['streams'])


def test_wide_sum_uses_accumulation():
    def build(b, v):
        parts = [ios.conv2d(b, [[v]], 6, (1, 1), act='identity') for _ in range(11)]
        ios.relu(b, [parts], is_exit=True)
    graph = single_op_graph((4, 6, 6), build)
    got, want = run_both(graph, 2)
    assert_close(got, want, 'sum of 11 values')


def test_sequential_units_and_folded_relu():
    def build(b, v):
        a = ios.relu_sep_conv(b, [[v]], 12, (3, 3), (2, 2), (1, 1))
        c = ios.relu_conv(b, [[a]], 9, (1, 1))
        d = ios.sep_conv(b, [[a]], 9, (5, 5), (1, 1), (2, 2))
        ios.relu_sep_conv(b, [[c, d]], 7, (3, 3), (1, 1), (1, 1), is_exit=True)
    graph = single_op_graph((8, 12, 12), build)
    for batch in (1, 2):
        got, want = run_both(graph, batch)
        assert_close(got, want, 'sequential units')


def separable_graph(in_shape, inputs, relu, oc, window, stride):
    """`inputs` 1x1 convolutions of the placeholder feed one (ReLU,) depth-wise, 1x1 unit whose output sits in a concat."""
    def build(b, v):
        parts = [ios.conv2d(b, [[v]], in_shape[0], (1, 1), act='identity') for _ in range(inputs)]
        pad = (window // 2, window // 2)
        make = ios.relu_sep_conv if relu else ios.sep_conv
        unit = make(b, [parts], oc, (window, window), (stride, stride), pad)
        other = ios.conv2d(b, [[unit]], 6, (1, 1))
        ios.identity(b, [[other], [unit]], is_exit=True)      # the unit writes into a channel window of this buffer
    return single_op_graph(in_shape, build)


def test_depthwise_kernel_adds_up_to_eight_inputs_in_its_loader():
    """(sum of k values,) (ReLU,) depth-wise convolution: no summing launch, no sum tensor (3 x 3 and 5 x 5 windows)."""
    for in_shape, inputs, relu, oc, window, stride, batch in [((312, 7, 7), 8, True, 312, 3, 1, 1), ((200, 9, 9), 3, True, 64, 3, 2, 2),
                                                              ((78, 28, 28), 2, True, 78, 3, 1, 2), ((21, 9, 9), 2, False, 33, 3, 2, 3),
                                                              ((176, 7, 7), 2, False, 176, 5, 1, 1), ((96, 8, 8), 5, True, 96, 5, 1, 3),
                                                              ((3, 6, 6), 7, True, 5, 5, 2, 1), ((64, 10, 10), 2, True, 64, 7, 1, 1)]:
        graph = separable_graph(in_shape, inputs, relu, oc, window, stride)
        ops = rt.plan_describe(graph, batch)
        kinds = [op['kind'] for op in ops]
        dw = [op for op in ops if op['kind'] == 'conv_depthwise']
        assert len(dw) == 1
        if window <= 5:
            assert dw[0]['inputs'] == inputs and 'nary' not in kinds and dw[0]['conv']['pre_relu'] == int(relu)
        else:
            assert dw[0]['inputs'] == 1 and kinds.count('nary') == 1      # 7 x 7 windows keep the summing launch
        x = np.random.default_rng(14).standard_normal((batch, *in_shape)).astype(np.float32)
        want = ios_oracle.run(graph, x)
        outs = {}
        for executor in ('streams', 'fused'):
            rt.set_option('executor', executor)
            outs[executor] = rt.graph_inference(graph, batch, x)
            assert_close(outs[executor], want, f'depth-wise sum {in_shape} k={inputs} {window}x{window} {executor}')
        np.testing.assert_array_equal(outs['fused'], outs['streams'])


def test_depthwise_sums_share_fused_launches_with_other_operators():
    """A stage whose groups hold depth-wise convolutions of sums (3 x 3, 5 x 5), a matrix-path convolution, a pool and a sum."""
    def build(b, v):
        a = ios.conv2d(b, [[v]], 20, (1, 1), act='identity')
        c = ios.conv2d(b, [[v]], 20, (1, 1), act='identity')
        u3 = ios.relu_sep_conv(b, [[a, c, v]], 24, (3, 3), (1, 1), (1, 1))
        u5 = ios.sep_conv(b, [[a, c]], 24, (5, 5), (1, 1), (2, 2))
        u7 = ios.relu_sep_conv(b, [[a, v]], 24, (7, 7), (1, 1), (3, 3))
        e = ios.conv2d(b, [[a]], 24, (3, 3), padding=(1, 1))
        f = ios.pool2d(b, [[c]], 'avg', (3, 3), (1, 1), (1, 1))
        s = ios.identity(b, [[a, c]])
        ios.identity(b, [[u3], [u5], [u7], [e], [f], [s]], is_exit=True)
    graph = single_op_graph((20, 14, 14), build)
    names = [n.name for n in graph.blocks[0].inner_nodes]
    graph.blocks[0].stages = [[[names[0]], [names[1]]], [[n] for n in names[2:8]], [[graph.blocks[0].exit_node.name]]]
    for batch in (1, 2):
        x = np.random.default_rng(13).standard_normal((batch, 20, 14, 14)).astype(np.float32)
        want = ios_oracle.run(graph, x)
        outs = {}
        for executor in ('streams', 'fused', 'fused_graph', 'graph'):
            rt.set_option('executor', executor)
            outs[executor] = rt.graph_inference(graph, batch, x)
            assert_close(outs[executor], want, f'{executor} batch {batch}')
        for executor in ('fused', 'fused_graph', 'graph'):
            np.testing.assert_array_equal(outs[executor], outs['streams'])


def test_passes_queued_back_to_back_give_the_result_of_a_single_pass():
    graph = ios.models.squeezenet_1_1(init_seed=0, init_scheme='he_normal_bias')
    graph.greedy_schedule(8)
    x = np.random.default_rng(3).standard_normal((2, *graph.enter_node.output_shape)).astype(np.float32)
    for executor in ('streams', 'fused', 'fused_graph'):
        rt.set_option('executor', executor)
        with rt.Session(graph, 2) as session:
            session.load_weights()
            session.set_input(x)
            session.run()
            single = session.output()
            for _ in range(7):
                session.enqueue()
            session.synchronize()
            np.testing.assert_array_equal(session.output(), single)
    assert_close(single, ios_oracle.run(graph, x), 'squeezenet batch 2')


def model_cases():
    # (id, constructor, batch, strict tolerance).  Seeded non-zero biases everywhere; RandWire in the folded-batch-norm
    # form its configuration describes; NASNet both under the He-normal initialisation its configuration names (scaled
    # tolerance, see the module docstring) and in the folded form (strict).
    return [
        ('sample', lambda: ios.models.sample_network(init_seed=0, init_scheme='he_normal_bias'), 1, True),
        ('squeezenet_1_1', lambda: ios.models.squeezenet_1_1(init_seed=0, init_scheme='he_normal_bias'), 1, True),
        ('inception_v3', lambda: ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias'), 1, True),
        ('randwire_small', lambda: ios.models.randwire_small(init_seed=0, init_scheme='bn_folded'), 1, True),
        ('nasnet_mobile', lambda: ios.models.nasnet_mobile(init_seed=0, init_scheme='he_normal_bias'), 1, False),
        ('nasnet_mobile_folded', lambda: ios.models.nasnet_mobile(init_seed=0, init_scheme='bn_folded'), 1, True),
        ('inception_v3_b4', lambda: ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias'), 4, True),
    ]


def strict_misses(got, want):
    """Elements outside |d| <= 1e-4 + 1e-3 |want|, and the largest error in units of the last place of the tensor's largest value."""
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    misses = int((err > ATOL + RTOL * np.abs(want.astype(np.float64))).sum())
    ulp = float(np.spacing(np.float32(np.abs(want).max()))) if want.size else 1.0
    return misses, float(err.max()) / ulp


@pytest.mark.parametrize('name,make,batch,strict', model_cases(), ids=[c[0] for c in model_cases()])
def test_network_matches_oracle_under_every_schedule_and_executor(name, make, batch, strict):
    """
    Outputs match the CPU oracle within tolerance for the sequential, greedy and dp_parallel schedules under
    every executor.  With the kernel configuration pinned (it otherwise depends on how many groups share a
    stage, which changes the summation order) all schedules and executors agree bit for bit.
    """
    graph = make()
    assert any(np.abs(conv.bias).max() > 0 for conv in graph.conv_nodes())
    graph.sequential_schedule()
    x = np.random.default_rng(1).standard_normal((batch, *graph.enter_node.output_shape)).astype(np.float32)
    want_all = ios_oracle.run(graph, x, keep_all=True)
    want = want_all[graph.exit_node.name]
    rt.set_option('arena_reuse', 0)      # node by node: every operator's output has to survive the pass
    with rt.Session(graph, batch) as session:
        session.load_weights()
        session.set_input(x)
        session.run()
        got = session.output()
        # every operator's output, node by node: names the first operator that goes wrong
        report = []
        absorbed = 0
        for node in list(graph.nodes())[1:]:
            try:
                tensor = session.tensor(node)
            except RuntimeError as error:
                # a sum that only the ReLU behind it reads (RandWire's last stage output) is added by that ReLU's launch
                # an average pool exchanged with the 1 x 1 convolution behind it (Inception's pool branches) has no tensor either:
                # the convolution's output, checked like every other node, covers both
                assert 'no materialised output' in str(error)
                assert (node.type == 'identity' and name.startswith('randwire')) or (node.type == 'pool' and name.startswith('inception'))
                absorbed += 1
                continue
            assert_close(tensor, want_all[node.name], f'{name}: node {node.name} ({node.type})', scaled=not strict)
            if not strict:
                misses, ulps = strict_misses(tensor, want_all[node.name])
                if misses:
                    report.append((node.name, misses, tensor.size, ulps))
        if not strict:
            # He-normal without normalisation: the misses of the unscaled formula are roundings at the tensor's scale
            print(f'{name}: {len(report)} operators with elements outside |d| <= 1e-4 + 1e-3|want| '
                  f'(worst: {max(report, key=lambda r: r[3]) if report else None}; node, elements, of, max error in ulps of the largest value)')
            assert all(ulps <= 64.0 for _, _, _, ulps in report), report
            # a regression that pushes more operators, or more than stray elements of one, past the unscaled formula
            # shows here even while every error stays within the scaled tolerance (152 operators, at most 0.13 % of a
            # tensor's elements, when this bound was written)
            assert len(report) <= 200, len(report)
            worst_share = max((misses / size for _, misses, size, _ in report), default=0.0)
            print(f'{name}: largest share of a tensor outside the unscaled formula: {worst_share:.5f}')
            assert worst_share <= 0.02, worst_share
    assert_close(got, want, name, scaled=not strict)
    assert np.isfinite(got).all() and np.abs(got).max() > 0
    assert absorbed == (1 if name.startswith('randwire') else 9 if name.startswith('inception') else 0)
    rt.set_option('arena_reuse', 1)      # everything below runs in the shared arena

    big = name.startswith(('randwire', 'nasnet'))
    greedy = make()
    greedy.greedy_schedule(4 if big else 8)
    if big:     # keep the pure-Python search short: small consecutive parts instead of whole cells
        for block in graph.blocks:
            block.parts = None
    optimized = ios.optimize(graph, batch, ios.AnalyticCostModel(), 'dp_parallel', max_group_size=2,
                             max_num_groups=4 if big else 8, max_part_size=10 if big else 100, compute_weight=True)
    assert any(len(stage) > 1 for block in optimized.blocks for stage in block.stages)

    def run_all(pinned):
        outs = {}
        for executor in ('streams', 'graph', 'fused', 'fused_graph'):
            rt.set_option('executor', executor)
            for label, g in (('sequential', graph), ('greedy', greedy), ('dp_parallel', optimized)):
                if label == 'sequential' and executor != 'streams':
                    continue
                with rt.Session(g, batch) as session:
                    session.load_weights()
                    session.set_input(x)
                    for _ in range(2):      # the second pass replays the captured graph
                        session.run()
                    outs[(executor, label)] = session.output()
                assert_close(outs[(executor, label)], want, f'{name} {executor} {label} pinned={pinned}', scaled=not strict)
        return outs

    run_all(pinned=False)
    rt.set_option('conv_variant', rt.device_info()['conv_variants'].index('wq_m32n16_w8_t16'))
    rt.set_option('conv_split_k', 2)
    outs = run_all(pinned=True)
    first = outs[('streams', 'sequential')]
    for key, value in outs.items():
        np.testing.assert_array_equal(value, first, err_msg=str(key))


@pytest.mark.parametrize('name,make', [
    ('sample', lambda: ios.models.sample_network(init_seed=0, init_scheme='he_normal_bias')),
    ('randwire_small', lambda: ios.models.randwire_small(init_seed=0, init_scheme='bn_folded')),
    ('nasnet_mobile_folded', lambda: ios.models.nasnet_mobile(init_seed=0, init_scheme='bn_folded')),
], ids=['sample', 'randwire_small', 'nasnet_mobile_folded'])
def test_network_with_measured_kernel_configurations_matches_oracle(name, make):
    """
    The configuration the latency figures of these networks are quoted on: kernel variants and split-K picked by
    measurement (not the closed form the rest of the suite pins), a parallel schedule, one fused launch per level
    replayed from a captured graph.  Strict tolerance against the CPU oracle, on the first pass and on replays.
    """
    graph = make()
    graph.sequential_schedule()
    x = np.random.default_rng(5).standard_normal((1, *graph.enter_node.output_shape)).astype(np.float32)
    want = ios_oracle.run(graph, x)
    graph.greedy_schedule(4 if name != 'sample' else 8)
    rt.set_option('autotune', 1)
    rt.set_option('executor', 'fused_graph')
    try:
        with rt.Session(graph, 1) as session:
            session.load_weights()
            session.set_input(x)
            outs = []
            for _ in range(3):
                session.run()
                outs.append(session.output())
            ops = session.describe()
        for got in outs:
            assert_close(got, want, f'{name} measured configurations, fused_graph')
            np.testing.assert_array_equal(got, outs[0])
        # the measured choice is in force: it differs from what the closed form picks for the same plan
        picked = [op['variant'] for op in ops if 'variant' in op]
        closed_form = [op['variant'] for op in rt.plan_describe(graph, 1) if 'variant' in op]
        assert len(picked) == len(closed_form) and picked != closed_form, picked
    finally:
        rt.set_option('autotune', 0)


@pytest.mark.parametrize('variant_name', ['x3w_m64n32_w4', 'x3w_m32n64_w4', 'x3w_m32n32_w8', 'x3w_m64n32_w2'])
def test_three_term_configurations_inside_fused_stage_launches(variant_name):
    """
    The three-term wave-split bodies are too heavy on registers for the fused stage kernels with six wavefronts per SIMD and run
    in a family of their own (256 and 512 threads, items in the table): parallel stages of Inception-v3 at batch 4 with one such
    configuration pinned for every convolution, against the oracle and bit for bit against the stream executor.
    """
    graph = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    graph.sequential_schedule()
    x = np.random.default_rng(2).standard_normal((4, *graph.enter_node.output_shape)).astype(np.float32)
    want = ios_oracle.run(graph, x)
    graph.greedy_schedule(8)
    rt.set_option('conv_variant', rt.device_info()['conv_variants'].index(variant_name))
    rt.set_option('conv_split_k', 1)
    outs = {}
    for executor in ('streams', 'fused', 'fused_graph'):
        rt.set_option('executor', executor)
        with rt.Session(graph, 4) as session:
            session.load_weights()
            session.set_input(x)
            for _ in range(2):
                session.run()
            outs[executor] = session.output()
            if executor == 'fused':
                kernels = {launch['kernel'] for launch in session.launches() if len(launch['ops']) > 1}
                threads = 512 if variant_name.endswith('w8') else 256
                assert f'fused_kernel_wide<{threads}>' in kernels, kernels
    assert_close(outs['streams'], want, variant_name)
    for executor in ('fused', 'fused_graph'):
        np.testing.assert_array_equal(outs[executor], outs['streams'], err_msg=executor)


# The rest of the reference's model zoo (python/ios/models/{alexnet,vgg,resnet}.py): chains, and residual networks whose
# additions are the two-operand `element` operator.  (id, constructor, batch, operators without a tensor of their own: the
# last convolution of a residual unit writes the sum, and the addition in front of a ReLU is part of that launch too)
ZOO = [
    ('alexnet', lambda: ios.models.alexnet(init_seed=0, init_scheme='he_normal_bias'), 2, 0),
    ('vgg_11', lambda: ios.models.vgg_11(init_seed=0, init_scheme='he_normal_bias'), 1, 0),
    ('vgg_16', lambda: ios.models.vgg_16(init_seed=0, init_scheme='he_normal_bias'), 1, 0),
    ('resnet18', lambda: ios.models.resnet18(init_seed=0, init_scheme='bn_folded'), 2, 8),
    ('resnet34', lambda: ios.models.resnet34(init_seed=0, init_scheme='bn_folded'), 1, 16),
    ('resnet50', lambda: ios.models.resnet50(init_seed=0, init_scheme='bn_folded'), 1, 32),
    # one stage of 320 nodes on the reference's own edge list (a fixture): sums of up to 33 values, in chunks of eight
    ('randwire_xlarge', lambda: ios.models.randwire_xlarge(init_seed=0, init_scheme='bn_folded', graph_file=os.path.join(
        os.path.dirname(__file__), 'golden', 'randwire_graphs', 'ws-320-20-0.75-x.txt')), 1, 1),
]


@pytest.mark.parametrize('name,make,batch,absorbed', ZOO, ids=[c[0] for c in ZOO])
def test_zoo_network_matches_oracle(name, make, batch, absorbed):
    graph = make()
    graph.sequential_schedule()
    x = np.random.default_rng(1).standard_normal((batch, *graph.enter_node.output_shape)).astype(np.float32)
    want_all = ios_oracle.run(graph, x, keep_all=True)
    want = want_all[graph.exit_node.name]
    assert np.isfinite(want).all() and 0 < np.abs(want).max() < 1e3
    rt.set_option('arena_reuse', 0)
    with rt.Session(graph, batch) as session:
        session.load_weights()
        session.set_input(x)
        session.run()
        missing = 0
        for node in list(graph.nodes())[1:]:
            try:
                tensor = session.tensor(node)
            except RuntimeError as error:
                assert 'no materialised output' in str(error) and node.type in ('element', 'conv', 'identity')
                missing += 1
                continue
            assert_close(tensor, want_all[node.name], f'{name}: node {node.name} ({node.type})')
        assert missing == absorbed
    rt.set_option('arena_reuse', 1)
    greedy = make()
    greedy.greedy_schedule(8)
    for executor in ('streams', 'fused', 'fused_graph'):
        rt.set_option('executor', executor)
        for label, g in (('sequential', graph), ('greedy', greedy)):
            with rt.Session(g, batch) as session:
                session.load_weights()
                session.set_input(x)
                for _ in range(2):
                    session.run()
                assert_close(session.output(), want, f'{name} {executor} {label}')


def test_every_form_of_the_fused_stage_kernel_runs_and_matches_the_oracle():
    """Launches of a fused stage carry their work items in the kernel-argument segment when they hold at most eight of them
    (one kernel for levels with matrix-path convolutions, one for levels of depth-wise convolutions, pools and sums) and read
    them from a table in device memory otherwise.  NASNet-A mobile under the greedy schedule uses all three forms; a stage of
    ten parallel 1x1 convolutions takes the table form because of its size."""
    graph = ios.models.nasnet_mobile(init_seed=0, init_scheme='he_normal_bias')
    graph.greedy_schedule(8)
    x = np.random.default_rng(5).standard_normal((1, *graph.enter_node.output_shape)).astype(np.float32)
    want = ios_oracle.run(graph, x)
    rt.set_option('executor', 'fused')
    with rt.Session(graph, 1) as session:
        session.load_weights()
        session.set_input(x)
        kernels = {launch['kernel'].split('<')[0] for launch in session.launches()}
        assert {'fused_kernel', 'fused_kernel_inline', 'fused_kernel_inline_direct'} <= kernels, kernels
        session.run()
        assert_close(session.output(), want, 'nasnet_mobile greedy')

    ios.reset_name()
    v = ios.placeholder((16, 12, 12))
    block = ios.Block(v.node)
    outs = [ios.conv2d(block, [[v]], 8 + i, (1, 1), (1, 1), (0, 0), 1, 'relu') for i in range(10)]
    out = ios.identity(block, [[o] for o in outs], is_exit=True)
    wide = Graph('ten_branches', v.node, [block])
    wide.init_weights(3, 'he_normal_bias')
    block.stages = [[[o.node.name] for o in outs], [[out.node.name]]]
    x = np.random.default_rng(6).standard_normal((2, 16, 12, 12)).astype(np.float32)
    want = ios_oracle.run(wide, x)
    with rt.Session(wide, 2) as session:
        session.load_weights()
        session.set_input(x)
        first = session.launches()[0]
        assert first['kernel'].startswith('fused_kernel<') and len(first['ops']) == 10, first
        session.run()
        assert_close(session.output(), want, 'ten parallel convolutions')


def test_activation_absorbs_the_combination_in_front_of_it():
    """add -> relu, mul -> tanh, three-way sum -> sigmoid become one launch each; a combination that somebody else reads, or
    that the activation reads in part, stays a launch of its own.  Results as in the oracle either way."""
    def build(b, v):
        a = ios.conv2d(b, [[v]], 8, (1, 1), act='identity')
        c = ios.conv2d(b, [[v]], 8, (3, 3), padding=(1, 1), act='identity')
        e1 = ios.addition(b, [[a, c]])
        r1 = ios.relu(b, [[e1]])                                   # absorbed
        e2 = ios.multiply(b, [[a, r1]])
        t2 = ios.activation(b, [[e2]], 'tanh', True)               # absorbed
        s3 = ios.identity(b, [[a, c, t2]])
        g3 = ios.sigmoid(b, [[s3]])                                # absorbed
        e4 = ios.addition(b, [[g3, c]])
        r4 = ios.relu(b, [[e4]])                                   # e4 has a second reader: kept
        e5 = ios.addition(b, [[r4, a]])
        r5 = ios.relu(b, [[Value(e5.node, 2, 6)]])                 # reads a slice: kept
        ios.identity(b, [[r4], [e4], [r5], [g3]], is_exit=True)
    graph = single_op_graph((6, 9, 9), build)
    for batch in (1, 3):
        ops = rt.plan_describe(graph, batch)
        assert sum(op['kind'] == 'nary' for op in ops) == 5 and sum(op['kind'] == 'unary' for op in ops) == 2
        x = np.random.default_rng(8).standard_normal((batch, 6, 9, 9)).astype(np.float32)
        want = ios_oracle.run(graph, x)
        for executor in ('streams', 'fused'):
            rt.set_option('executor', executor)
            assert_close(rt.graph_inference(graph, batch, x), want, f'absorbed combinations, {executor}, batch {batch}')


@pytest.mark.parametrize('seed,large', [(seed, False) for seed in range(60)] + [(seed, True) for seed in range(16)])
def test_random_network_matches_oracle(seed, large):
    """Seeded random wiring of every operator kind under a random schedule (tests/random_graphs.py; `large`: 24-190 channels
    on 20-44 pixel sides): every tensor the plan materialises and the result agree with the oracle, under the stream and the
    fused executors, with and without arena reuse."""
    import random_graphs
    graph, batch, built = random_graphs.random_graph(seed, large)
    x = np.random.default_rng(seed).standard_normal((batch, *graph.enter_node.output_shape)).astype(np.float32)
    want_all = ios_oracle.run(graph, x, keep_all=True)
    want = ios_oracle.run(built, x)      # (the graph as built: a merge search must not change the function)
    rt.set_option('arena_reuse', 0)
    with rt.Session(graph, batch) as session:
        session.load_weights()
        session.set_input(x)
        session.run()
        compared = 0
        for node in list(graph.nodes())[1:]:
            try:
                tensor = session.tensor(node)
            except RuntimeError as error:
                assert 'no materialised output' in str(error)
                continue
            assert_close(tensor, want_all[node.name], f'seed {seed}: node {node.name} ({node.type})', scaled=True)
            compared += 1
        assert compared >= len(list(graph.nodes())) // 2
    rt.set_option('arena_reuse', 1)
    for executor in ('streams', 'fused', 'fused_graph'):
        rt.set_option('executor', executor)
        with rt.Session(graph, batch) as session:
            session.load_weights()
            session.set_input(x)
            for _ in range(2):
                session.run()
            assert_close(session.output(), want, f'seed {seed}, {executor}', scaled=True)


@pytest.mark.parametrize('seed', range(100, 124))
def test_random_network_through_the_other_entry_points(seed):
    """The same random networks through the entry point that allocates nothing (bit-identical), in the reduced-precision
    modes (error of the operand rounding) and through graph / block / stage latency under the stream and the fused executor."""
    import random_graphs
    graph, batch, built = random_graphs.random_graph(seed)
    x = np.random.default_rng(seed).standard_normal((batch, *graph.enter_node.output_shape)).astype(np.float32)
    want = ios_oracle.run(built, x)
    rt.set_option('executor', 'fused')
    plain = rt.graph_inference(graph, batch, x)
    assert_close(plain, want, f'seed {seed}', scaled=True)
    np.testing.assert_array_equal(rt.graph_inference(graph, batch, x, no_alloc=True), plain)
    for precision in ('bf16', 'fp16'):
        rt.set_option('precision', precision)
        assert_close_reduced(rt.graph_inference(graph, batch, x), want, f'seed {seed}, {precision}')
    rt.set_option('precision', 'fp32')
    stages = sum(len(block.stages) for block in graph.blocks)
    for executor in ('streams', 'fused'):
        rt.set_option('executor', executor)
        total, per_stage = rt.graph_latency(graph, batch, 0, 1, 2, profile_stage=True)
        assert len(total) == 2 and len(per_stage) == 2 * stages and min(total) > 0
        for block in graph.blocks:
            assert min(rt.block_latency(block, batch, 0, 1, 1)) > 0
            names = {node.name: node for node in block.inner_nodes + [block.exit_node]}
            for stage in block.stages:
                assert min(rt.stage_latency([[names[name] for name in group] for group in stage], batch, 0, 1, 1)) > 0


def test_inception_batch_16_under_the_schedule_searched_at_that_batch():
    """
    The middle point of the batch sweep, the way the benchmark runs it: dp_parallel schedule searched with on-device stage
    measurements at batch 16 (r = 1, s = 8), measured kernel configurations, fused launches replayed from a hipGraph;
    sampled images against the oracle, which sees those images only.
    """
    batch = 16
    graph = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    rt.set_option('autotune', 1)
    rt.set_option('executor', 'fused')
    try:
        optimized = ios.optimize(graph, batch_size=batch, opt_type='dp_parallel', compute_weight=True, warmup=1, number=2, repeat=1,
                                 max_group_size=1, max_num_groups=8)
        assert any(len(stage) > 1 for block in optimized.blocks for stage in block.stages)
        x = np.random.default_rng(6).standard_normal((batch, *graph.enter_node.output_shape)).astype(np.float32)
        x[11] = x[3]
        sample = [0, 3, 9, 15]
        graph.sequential_schedule()
        want = ios_oracle.run(graph, x[sample])
        outs = {}
        for executor, g in (('fused_graph', optimized), ('fused', optimized), ('fused_graph', graph)):
            rt.set_option('executor', executor)
            with rt.Session(g, batch) as session:
                session.load_weights()
                session.set_input(x)
                for _ in range(2):
                    session.run()
                got = session.output()
            assert got.shape[0] == batch and np.isfinite(got).all()
            assert_close(got[sample], want, f'inception batch 16 {executor} {"dp_parallel" if g is optimized else "sequential"}')
            np.testing.assert_array_equal(got[11], got[3])
    finally:
        rt.set_option('autotune', 0)
        rt.set_option('executor', 'streams')


@pytest.mark.parametrize('name', ['1', '16', '32', '64', '128', 'k80', 'v100'])
def test_reference_schedule_files_run_and_match_the_plain_model(name):
    """
    The reference's own optimised schedules (experiments/specialization/schedules/*.json: merged convolutions read through
    channel slices, up to five groups per stage), loaded unchanged and run at the batch size each was tuned for
    (experiments/specialization/main.py:43-48).  With the plain model's weights stacked into the merged convolutions the
    result must equal the plain model's on the oracle.
    """
    import reference_schedules
    batch = reference_schedules.TUNED_BATCH[name]
    plain = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    plain.sequential_schedule()
    graph = reference_schedules.load(name)
    reference_schedules.adopt_weights(graph, plain)
    x = np.random.default_rng(8).standard_normal((batch, 3, 299, 299)).astype(np.float32)
    sample = sorted({0, batch // 2, batch - 1})
    want = ios_oracle.run(plain, x[sample])
    for executor in ('fused', 'streams'):
        rt.set_option('executor', executor)
        got = rt.graph_inference(graph, batch, x)
        assert got.shape == (batch, 2048, 1, 1)
        assert_close(got[sample], want, f'reference schedule {name}.json at batch {batch}, {executor}')
    latency = rt.graph_latency(graph, batch, warmup=1, number=2, repeat=2)
    assert len(latency) == 2 and all(v > 0 for v in latency)


def test_large_batch_parallel_stages_with_measured_kernel_configurations():
    """
    At batch 32 no kernel configuration fits the share of the device a group of a parallel stage is budgeted,
    so the tuner falls back; whatever it picks must be able to run inside the fused stage launch.
    """
    graph = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    graph.greedy_schedule(8)
    batch = 32
    x = np.random.default_rng(4).standard_normal((batch, *graph.enter_node.output_shape)).astype(np.float32)
    want = ios_oracle.run(graph, x)
    rt.set_option('autotune', 1)
    try:
        for executor in ('fused', 'streams'):
            rt.set_option('executor', executor)
            with rt.Session(graph, batch) as session:
                session.load_weights()
                session.set_input(x)
                session.run()
                assert_close(session.output(), want, f'inception batch {batch} {executor}')
    finally:
        rt.set_option('autotune', 0)


def test_batch_64_images_are_independent_and_match_the_oracle():
    """
    The largest configuration of the batch sweep with the measured kernel configurations the benchmark runs: an
    image's output depends on that image alone, so a sample of the 64 outputs is checked against the oracle run
    on those images only, and two identical images inside the batch must give identical outputs.
    """
    graph = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    graph.sequential_schedule()
    batch = 64
    x = np.random.default_rng(9).standard_normal((batch, *graph.enter_node.output_shape)).astype(np.float32)
    x[41] = x[5]
    sample = [0, 5, 17, 63]
    want = ios_oracle.run(graph, x[sample])
    rt.set_option('autotune', 1)
    rt.set_option('executor', 'fused_graph')
    try:
        with rt.Session(graph, batch) as session:
            session.load_weights()
            session.set_input(x)
            session.run()
            got = session.output()
    finally:
        rt.set_option('autotune', 0)
        rt.set_option('executor', 'streams')
    assert got.shape[0] == batch and np.isfinite(got).all()
    assert_close(got[sample], want, 'inception batch 64, sampled images')
    np.testing.assert_array_equal(got[41], got[5])


def matrix_path_convs(graph, batch):
    return frozenset(op['node'] for op in rt.plan_describe(graph, batch) if op['kind'] == 'conv_mfma')


def assert_close_reduced(got, want, what=''):
    """bfloat16 operands carry 8 bits of mantissa: 2^-8 per operand against the fp32 result, taken at the tensor's scale."""
    scale = max(1.0, float(np.abs(want).max()))
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert err.max() <= 3e-2 * scale, f'{what}: max abs err {err.max():.3e} at scale {scale:.3e}'


REDUCED = [('bf16', 'wb_', 'bf16_convs'), ('fp16', 'wh_', 'fp16_convs')]


@pytest.mark.parametrize('mode', REDUCED, ids=[m[0] for m in REDUCED])
@pytest.mark.parametrize('case', [c for c in CONVS if c[5] == 1])
def test_reduced_precision_conv_matches_the_rounding_oracle(case, mode):
    """precision=bf16 / fp16: bit-level agreement is not expected (summation order), but against an oracle that rounds the
    same operands to bfloat16 / half the fp32 tolerance holds; against the fp32 oracle the error is that of the rounding."""
    precision, _, oracle_key = mode
    in_shape, oc, k, s, p, g, act, batch = case
    graph = single_op_graph(in_shape, lambda b, v: ios.conv2d(b, [[v]], oc, k, s, p, g, act, is_exit=True))
    x = np.random.default_rng(1).standard_normal((batch, *in_shape)).astype(np.float32)
    rt.set_option('precision', precision)
    convs = matrix_path_convs(graph, batch)
    assert convs, 'expected a matrix-path convolution'
    got = rt.graph_inference(graph, batch, x)
    assert_close(got, ios_oracle.run(graph, x, **{oracle_key: convs}), f'{precision} conv {case}')
    assert_close_reduced(got, ios_oracle.run(graph, x), f'{precision} conv {case} against fp32')
    rt.set_option('precision', 'fp32')
    assert not np.array_equal(got, rt.graph_inference(graph, batch, x))     # the mode really changes the arithmetic


@pytest.mark.parametrize('mode', REDUCED, ids=[m[0] for m in REDUCED])
def test_every_reduced_precision_kernel_configuration(mode):
    precision, prefix, oracle_key = mode
    names = rt.device_info()['conv_variants']
    rt.set_option('precision', precision)
    tried = 0
    for index, name in enumerate(names):
        if not name.startswith(prefix):
            continue
        tried += 1
        rt.set_option('conv_variant', index)
        for split in (1, 3):
            rt.set_option('conv_split_k', split)
            for in_shape, oc, k, s, p, batch in [((72, 19, 19), 88, (3, 3), (1, 1), (1, 1), 2),
                                                  ((200, 8, 8), 136, (1, 1), (1, 1), (0, 0), 1),
                                                  ((20, 37, 37), 24, (5, 5), (2, 2), (2, 2), 1)]:
                graph = single_op_graph(in_shape, lambda b, v: ios.conv2d(b, [[v]], oc, k, s, p, 1, 'relu', is_exit=True))
                x = np.random.default_rng(1).standard_normal((batch, *in_shape)).astype(np.float32)
                got = rt.graph_inference(graph, batch, x)
                want = ios_oracle.run(graph, x, **{oracle_key: matrix_path_convs(graph, batch)})
                assert_close(got, want, f'{name} split {split} conv {in_shape}->{oc} {k}')
                np.testing.assert_array_equal(got, rt.graph_inference(graph, batch, x))
    assert tried >= 10


@pytest.mark.parametrize('mode', REDUCED, ids=[m[0] for m in REDUCED])
def test_reduced_precision_network_under_parallel_schedules(mode):
    precision, _, oracle_key = mode
    graph = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    graph.sequential_schedule()
    greedy = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    greedy.greedy_schedule(8)
    x = np.random.default_rng(1).standard_normal((2, *graph.enter_node.output_shape)).astype(np.float32)
    rt.set_option('precision', precision)
    convs = matrix_path_convs(graph, 2)
    assert len(convs) == 94
    want = ios_oracle.run(graph, x, **{oracle_key: convs})
    want_fp32 = ios_oracle.run(graph, x)
    for executor, g in (('streams', graph), ('fused', greedy), ('fused_graph', greedy)):
        rt.set_option('executor', executor)
        with rt.Session(g, 2) as session:
            session.load_weights()
            session.set_input(x)
            for _ in range(2):
                session.run()
            got = session.output()
        # 94 layers deep, a different rounding of one operand (summation order before it) can flip a 16-bit rounding
        # downstream: the rounding oracle is matched at the rounding tolerance, a little tighter than the fp32 one
        assert_close_reduced(got, want, f'{precision} inception {executor}')
        assert_close_reduced(got, want_fp32, f'{precision} inception {executor} against fp32')
        assert np.abs(got - want).max() <= np.abs(got - want_fp32).max() * 1.5 + 1e-4


def test_merged_convolutions_match_unmerged():
    graph = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    merged = ios.optimize(graph, 1, ios.AnalyticCostModel(launch=1.0, rate=2e7, sync=1.5), 'dp_parallel_merge',
                          compute_weight=True)
    assert any(' ' in node.hint_name for node in merged.nodes())
    x = np.random.default_rng(1).standard_normal((2, 3, 299, 299)).astype(np.float32)
    graph.sequential_schedule()
    want = ios_oracle.run(graph, x)
    for batch in (1, 2):    # channel slices of merged convolutions are read in place at any batch size
        got = rt.graph_inference(merged, batch, x[:batch])
        assert_close(got, want[:batch], f'merged graph batch {batch}')


def test_latency_entry_points():
    graph = ios.models.sample_network()
    graph.sequential_schedule()
    lat = rt.graph_latency(graph, batch_size=1, warmup=1, number=2, repeat=3)
    assert len(lat) == 3 and all(0 < v < 1000 for v in lat)
    lat, stages = rt.graph_latency(graph, batch_size=1, warmup=1, number=2, repeat=3, profile_stage=True)
    table = np.array(stages).reshape(3, -1)
    assert table.shape == (3, 5) and (table >= 0).all()
    assert table.sum(axis=1) == pytest.approx(np.array(lat), rel=0.05, abs=0.02)
    blk = rt.block_latency(graph.blocks[0], 1, 1, 2, 3)
    assert len(blk) == 3 and all(v > 0 for v in blk)
    nodes = graph.blocks[0].inner_nodes
    one = rt.stage_latency([[nodes[0]]], 1, 1, 2, 3)
    two = rt.stage_latency([[nodes[0], nodes[3]], [nodes[1]], [nodes[2]]], 1, 1, 2, 3)
    assert len(one) == 3 and len(two) == 3 and all(v > 0 for v in one + two)
    with pytest.raises(RuntimeError):
        rt.stage_latency([[nodes[0]]], 1, 1, 2, 3, profile_stage=True)


def test_optimize_with_measured_cost_model_on_sample_net():
    graph = ios.models.sample_network(init_seed=0, init_scheme='he_normal_bias')
    optimized = ios.optimize(graph, batch_size=1, opt_type='dp_parallel', compute_weight=True, warmup=1, number=2, repeat=2)
    names = sorted(n for stage in optimized.blocks[0].stages for group in stage for n in group)
    assert names == ['1', '2', '3', '4', '5']
    x = np.random.default_rng(0).standard_normal((1, 375, 15, 15))      # float64 on purpose: the glue converts
    got = rt.graph_inference(optimized, 1, x)
    graph.sequential_schedule()
    assert_close(got, ios_oracle.run(graph, x.astype(np.float32)), 'optimized sample net')


def test_measured_search_with_groups_of_one_operator_under_the_fused_executor():
    """The pruning the benchmark uses (r = 1, s = 8): stages are sets of independent operators, one fused launch each."""
    rt.set_option('executor', 'fused')
    rt.set_option('autotune', 1)
    try:
        for make in (ios.models.squeezenet_1_1, ios.models.inception_v3):
            graph = make(init_seed=0, init_scheme='he_normal_bias')
            optimized = ios.optimize(graph, batch_size=1, opt_type='dp_parallel', compute_weight=True, warmup=1, number=2, repeat=1,
                                     max_group_size=1, max_num_groups=8)
            stages = [stage for block in optimized.blocks for stage in block.stages]
            assert all(len(group) == 1 for stage in stages for group in stage) and all(len(stage) <= 8 for stage in stages)
            assert any(len(stage) > 1 for stage in stages)
            assert sorted(n for stage in stages for group in stage for n in group) == sorted(n.name for n in graph.nodes() if n is not graph.enter_node)
            x = np.random.default_rng(2).standard_normal((1, *graph.enter_node.output_shape)).astype(np.float32)
            graph.sequential_schedule()
            want = ios_oracle.run(graph, x)
            for executor in ('fused', 'fused_graph'):
                rt.set_option('executor', executor)
                assert_close(rt.graph_inference(optimized, 1, x), want, f'{graph.name} r=1 {executor}')
            rt.set_option('executor', 'fused')
    finally:
        rt.set_option('autotune', 0)


def test_calls_from_two_host_threads_are_serialised():
    """The library keeps process-wide state; its entry points take a lock, so concurrent callers get correct results."""
    import threading
    graph = ios.models.squeezenet_1_1(init_seed=0, init_scheme='he_normal_bias')
    graph.greedy_schedule(8)
    x = np.random.default_rng(3).standard_normal((1, *graph.enter_node.output_shape)).astype(np.float32)
    want = ios_oracle.run(graph, x)
    results, errors = {}, []

    def worker(index):
        try:
            for _ in range(3):
                results[index] = rt.graph_inference(graph, 1, x)
                latency = rt.graph_latency(graph, 1, warmup=1, number=2, repeat=2)
                assert len(latency) == 2 and all(v > 0 for v in latency)
        except Exception as error:   # noqa: BLE001 - reported by the main thread
            errors.append(error)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for index in range(2):
        assert_close(results[index], want, f'thread {index}')


def test_errors_are_reported_not_fatal():
    graph = ios.models.sample_network(init_seed=0)
    with pytest.raises(RuntimeError, match='no schedule'):
        rt._latency_call('graph_latency', [__import__('json').dumps(graph.export_config())], 1, 1, 1, 1, 1, False)
    graph.blocks[0].stages = [[['1'], ['4']], [['2'], ['3']], [['5']]]
    with pytest.raises(RuntimeError, match='not topological'):
        rt.graph_latency(graph, 1, 1, 1, 1)
    graph.blocks[0].stages = [[[str(i)] for i in range(1, 5)] * 5, [['5']]]
    with pytest.raises(RuntimeError):
        rt.graph_latency(graph, 1, 1, 1, 1)
    graph.sequential_schedule()
    x = np.zeros((1, 375, 15, 15), np.float32)
    with pytest.raises(ValueError):
        rt.graph_inference(graph, 2, x)
    assert rt.graph_inference(graph, 1, x).shape == (1, 1875, 15, 15)     # still alive after the failures
