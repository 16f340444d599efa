"""
Pins the CPU oracle: the torch-backed routines of oracle/ios_oracle.py against explicit-loop formulas
(oracle/brute.py), against the plain-C restatement (oracle/conv_ref.c) and against closed forms.
Tolerance: the oracle computes in float32, the brute-force versions accumulate in float64, so agreement
is required to rel 1e-5 / abs 1e-5 on O(1) data.
"""
import numpy as np
import pytest
import torch

from oracle import brute, c_oracle, ios_oracle

RTOL, ATOL = 1e-5, 1e-5

CONV_CASES = [
    # n, ic, h, w, oc, kernel, stride, padding, groups, act
    (1, 3, 7, 7, 4, (3, 3), (1, 1), (1, 1), 1, 'relu'),
    (2, 4, 9, 8, 6, (3, 3), (2, 2), (0, 0), 1, 'identity'),
    (1, 4, 8, 8, 4, (1, 7), (1, 1), (0, 3), 1, 'relu'),
    (1, 4, 8, 8, 4, (7, 1), (1, 1), (3, 0), 1, 'tanh'),
    (2, 6, 6, 6, 6, (3, 3), (1, 1), (1, 1), 6, 'identity'),     # depthwise
    (1, 6, 7, 7, 6, (5, 5), (2, 2), (2, 2), 6, 'identity'),     # depthwise strided
    (1, 8, 5, 5, 4, (3, 3), (1, 1), (1, 1), 2, 'sigmoid'),      # grouped
    (1, 5, 6, 6, 7, (1, 1), (2, 2), (0, 0), 1, 'identity'),     # strided 1x1
    (1, 2, 5, 7, 3, (5, 5), (1, 1), (2, 2), 1, 'relu'),
]


def _conv_inputs(case, seed=0):
    n, ic, h, w, oc, k, s, p, g, act = case
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, ic, h, w)).astype(np.float32)
    wt = rng.standard_normal((oc, ic // g, *k)).astype(np.float32)
    b = rng.standard_normal(oc).astype(np.float32)
    return x, wt, b


def _oracle_conv(x, wt, b, s, p, g, act):
    return ios_oracle.conv2d(torch.from_numpy(x), torch.from_numpy(wt), torch.from_numpy(b), s, p, g, act).numpy()


@pytest.mark.parametrize('case', CONV_CASES)
def test_conv_matches_brute_force_and_c(case):
    n, ic, h, w, oc, k, s, p, g, act = case
    x, wt, b = _conv_inputs(case)
    got = _oracle_conv(x, wt, b, s, p, g, act)
    want = brute.conv2d(x, wt, b, s, p, g, act)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(c_oracle.conv2d(x, wt, b, s, p, g, act), want, rtol=RTOL, atol=ATOL)


def test_conv_medium_matches_c():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((2, 48, 35, 35)).astype(np.float32)
    wt = (rng.standard_normal((64, 48, 5, 5)) / 35.0).astype(np.float32)
    b = rng.standard_normal(64).astype(np.float32)
    np.testing.assert_allclose(_oracle_conv(x, wt, b, (1, 1), (2, 2), 1, 'relu'),
                               c_oracle.conv2d(x, wt, b, (1, 1), (2, 2), 1, 'relu'), rtol=1e-4, atol=1e-4)


def test_conv_1x1_is_matrix_product():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 16, 5, 6)).astype(np.float32)
    wt = rng.standard_normal((8, 16, 1, 1)).astype(np.float32)
    b = rng.standard_normal(8).astype(np.float32)
    want = np.einsum('oc,nchw->nohw', wt[:, :, 0, 0].astype(np.float64), x.astype(np.float64)) + b[None, :, None, None]
    np.testing.assert_allclose(_oracle_conv(x, wt, b, (1, 1), (0, 0), 1, 'identity'), want, rtol=RTOL, atol=ATOL)


def test_conv_delta_kernel_is_shift():
    # a 3x3 kernel with a single one at (i, j) shifts the image by (i-1, j-1) with zero fill (cross-correlation)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((1, 1, 6, 6)).astype(np.float32)
    for i in range(3):
        for j in range(3):
            wt = np.zeros((1, 1, 3, 3), dtype=np.float32)
            wt[0, 0, i, j] = 1.0
            got = _oracle_conv(x, wt, np.zeros(1, np.float32), (1, 1), (1, 1), 1, 'identity')
            padded = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
            np.testing.assert_array_equal(got, padded[:, :, i:i + 6, j:j + 6])


def test_conv_linearity_and_group_block_diagonal():
    rng = np.random.default_rng(4)
    x1 = rng.standard_normal((1, 6, 7, 7)).astype(np.float32)
    x2 = rng.standard_normal((1, 6, 7, 7)).astype(np.float32)
    wt = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)   # groups = 2
    zero = np.zeros(4, np.float32)
    f = lambda x: _oracle_conv(x, wt, zero, (1, 1), (1, 1), 2, 'identity')
    np.testing.assert_allclose(f(x1 + 2 * x2), f(x1) + 2 * f(x2), rtol=1e-4, atol=1e-4)
    dense = np.zeros((4, 6, 3, 3), dtype=np.float32)
    dense[:2, :3] = wt[:2]
    dense[2:, 3:] = wt[2:]
    np.testing.assert_allclose(f(x1), _oracle_conv(x1, dense, zero, (1, 1), (1, 1), 1, 'identity'), rtol=1e-5, atol=1e-5)


POOL_CASES = [
    ('max', (3, 3), (2, 2), (0, 0), (1, 3, 9, 9)),
    ('max', (3, 3), (2, 2), (1, 1), (2, 2, 8, 7)),
    ('avg', (3, 3), (1, 1), (1, 1), (1, 3, 6, 6)),
    ('avg', (3, 3), (2, 2), (1, 1), (1, 2, 7, 7)),
    ('max', (2, 2), (2, 2), (0, 0), (1, 2, 6, 6)),
    ('global_avg', (1, 1), (1, 1), (0, 0), (2, 5, 8, 8)),
    ('global_max', (1, 1), (1, 1), (0, 0), (1, 3, 4, 5)),
]


@pytest.mark.parametrize('case', POOL_CASES)
def test_pool_matches_brute_force_and_c(case):
    pool_type, k, s, p, shape = case
    x = np.random.default_rng(5).standard_normal(shape).astype(np.float32)
    # negative data everywhere makes a max pool that wrongly includes zero padding fail
    x_neg = -np.abs(x) - 1.0
    for data in (x, x_neg):
        got = ios_oracle.pool2d(torch.from_numpy(data), pool_type, k, s, p).numpy()
        want = brute.pool2d(data, pool_type, k, s, p)
        assert got.shape == want.shape
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
        np.testing.assert_allclose(c_oracle.pool2d(data, pool_type, k, s, p), want, rtol=RTOL, atol=ATOL)


def test_avg_pool_counts_padding():
    x = np.ones((1, 1, 4, 4), dtype=np.float32)
    got = ios_oracle.pool2d(torch.from_numpy(x), 'avg', (3, 3), (1, 1), (1, 1)).numpy()
    assert got[0, 0, 0, 0] == pytest.approx(4.0 / 9.0)      # corner: 4 real elements, divisor stays 9
    assert got[0, 0, 0, 1] == pytest.approx(6.0 / 9.0)
    assert got[0, 0, 1, 1] == pytest.approx(1.0)


def test_global_avg_is_mean():
    x = np.random.default_rng(6).standard_normal((2, 7, 8, 8)).astype(np.float32)
    got = ios_oracle.pool2d(torch.from_numpy(x), 'global_avg', (1, 1), (1, 1), (0, 0)).numpy()
    np.testing.assert_allclose(got[:, :, 0, 0], x.mean(axis=(2, 3)), rtol=1e-5, atol=1e-6)


def test_input_algebra_sum_concat_slice_and_mul():
    rng = np.random.default_rng(7)
    a = rng.standard_normal((2, 6, 3, 3)).astype(np.float32)
    b = rng.standard_normal((2, 4, 3, 3)).astype(np.float32)
    outs = {'a': torch.from_numpy(a), 'b': torch.from_numpy(b)}
    inputs = [[['a', 0, 4], ['b', 0, 4]], [['a', 2, 6]]]
    got = ios_oracle.gather_input(inputs, outs).numpy()
    want = np.concatenate([a[:, 0:4] + b, a[:, 2:6]], axis=1)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)
    got_mul = ios_oracle.gather_input([[['a', 0, 4], ['b', 0, 4]]], outs, multiply=True).numpy()
    np.testing.assert_allclose(got_mul, a[:, 0:4] * b, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(brute.gather_input(inputs, {'a': a, 'b': b}), want, rtol=1e-6, atol=1e-6)


def test_graph_interpreter_on_small_graph_matches_brute_force():
    import ios
    ios.reset_name()
    v = ios.placeholder((4, 6, 6))
    block = ios.Block(v.node)
    c1 = ios.conv2d(block, [[v]], 6, (3, 3), (1, 1), (1, 1), act='relu')
    c2 = ios.conv2d(block, [[v]], 6, (1, 1), act='identity')
    p = ios.pool2d(block, [[v]], 'avg', (3, 3), (1, 1), (1, 1))
    s = ios.sep_conv(block, [[c1, c2]], 5, (3, 3), (2, 2), (1, 1))
    r = ios.relu(block, [[p]])
    m = ios.pool2d(block, [[r], [Value_slice(c1, 1, 3)]], 'max', (3, 3), (2, 2), (1, 1))
    ios.identity(block, [[s], [m]], is_exit=True)
    graph = ios.Graph('tiny', v.node, [block])
    graph.init_weights(seed=11, scheme='he_normal')
    x = np.random.default_rng(8).standard_normal((2, 4, 6, 6)).astype(np.float32)
    got = ios_oracle.run(graph, x, keep_all=True)

    outs = {'0': x.astype(np.float64)}

    def ev(node):
        if node.type == 'sequential':
            for child in node.nodes:
                ev(child)
            outs[node.name] = outs[node.nodes[-1].name]
            return
        xin = brute.gather_input([[v.export_config() for v in t] for t in node.inputs], outs)
        if node.type == 'conv':
            y = brute.conv2d(xin, node.weight, node.bias, node.stride, node.padding, node.groups, node.act)
        elif node.type == 'pool':
            y = brute.pool2d(xin, node.pool_type, node.kernel, node.stride, node.padding)
        elif node.type == 'relu':
            y = np.maximum(xin, 0)
        else:
            y = xin
        outs[node.name] = y

    for node in list(graph.nodes())[1:]:
        ev(node)
    for name, want in outs.items():
        np.testing.assert_allclose(got[name], want, rtol=1e-4, atol=1e-5, err_msg=f'node {name}')
    assert got[graph.exit_node.name].shape == (2, 11, 3, 3)


def Value_slice(value, begin, end):
    from ios.ir import Value
    return Value(value.node, begin, end)


def test_bf16_rounding_is_round_to_nearest_even():
    """The oracle's bfloat16 view of an operand against the bit-level definition (add 0x7fff + lsb, truncate)."""
    import torch
    rng = np.random.default_rng(11)
    x = np.concatenate([rng.standard_normal(4096).astype(np.float32) * 10.0 ** rng.integers(-6, 6, 4096),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.0e38, -2.5e-39], dtype=np.float32)]).astype(np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    want = (((bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000) & 0xFFFFFFFF).astype(np.uint32).view(np.float32)
    got = ios_oracle.to_bf16(torch.from_numpy(x)).numpy()
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


def test_fp16_rounding_is_ieee_half_round_to_nearest_even():
    """The oracle's half view of an operand against numpy's float16 (an independent implementation) and known cases."""
    import torch
    rng = np.random.default_rng(12)
    x = np.concatenate([rng.standard_normal(4096).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 4096),
                        np.array([0.0, -0.0, 1.0, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65504.0, 65519.9, 65520.0, -1e6, 6e-8, 2.9e-8],
                                 dtype=np.float32)]).astype(np.float32)
    got = ios_oracle.to_fp16(torch.from_numpy(x)).numpy()
    with np.errstate(over='ignore'):
        want = x.astype(np.float16).astype(np.float32)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    known = ios_oracle.to_fp16(torch.tensor([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65519.9, 65520.0, 2.9e-8])).numpy()
    # ties go to the even mantissa; 65520 is the first value that rounds to infinity; below half the smallest subnormal: zero
    np.testing.assert_array_equal(known, np.array([1.0, 1.0 + 2.0 ** -9, 65504.0, np.inf, 0.0], dtype=np.float32))
    # a convolution named in fp16_convs sees exactly those operands
    import ios
    ios.reset_name()
    v = ios.placeholder((4, 5, 5))
    block = ios.Block(v.node)
    ios.conv2d(block, [[v]], 6, (3, 3), (1, 1), (1, 1), 1, 'identity', is_exit=True)
    graph = ios.Graph('h', v.node, [block])
    graph.init_weights(seed=3, scheme='he_normal_bias')
    conv = graph.conv_nodes()[0]
    xin = rng.standard_normal((2, 4, 5, 5)).astype(np.float32)
    got = ios_oracle.run(graph, xin, fp16_convs={conv.name})
    rounded = ios.Graph.from_config(graph.export_config())
    rounded.conv_nodes()[0].weight = conv.weight.astype(np.float16).astype(np.float32)
    rounded.conv_nodes()[0].bias = conv.bias
    want = ios_oracle.run(rounded, xin.astype(np.float16).astype(np.float32))
    np.testing.assert_array_equal(got, want)
    assert not np.array_equal(got, ios_oracle.run(graph, xin))


def _golden_vectors():
    import os
    import sys
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')
    sys.path.insert(0, golden)
    import make_operator_vectors as spec
    return spec, np.load(os.path.join(golden, 'operator_vectors.npz'))


def test_committed_operator_vectors_pin_the_oracle_and_the_c_restatement():
    """tests/golden/operator_vectors.npz holds inputs and brute-force outputs; both oracles must reproduce them."""
    spec, data = _golden_vectors()
    for name, shape, oc, kernel, stride, padding, groups, act in spec.CONVS:
        x, w, b, want = (data[f'{name}.{k}'] for k in 'xwby')
        assert x.shape == tuple(shape) and want.dtype == np.float32
        np.testing.assert_allclose(_oracle_conv(x, w, b, stride, padding, groups, act), want, rtol=RTOL, atol=ATOL, err_msg=name)
        np.testing.assert_allclose(c_oracle.conv2d(x, w, b, stride, padding, groups, act), want, rtol=RTOL, atol=ATOL, err_msg=name)
    for name, shape, pool_type, kernel, stride, padding in spec.POOLS:
        x, want = data[f'{name}.x'], data[f'{name}.y']
        got = ios_oracle.pool2d(torch.from_numpy(x), pool_type, kernel, stride, padding).numpy()
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL, err_msg=name)
        np.testing.assert_allclose(c_oracle.pool2d(x, pool_type, kernel, stride, padding), want, rtol=RTOL, atol=ATOL, err_msg=name)
