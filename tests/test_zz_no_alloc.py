"""
graph_inference_no_alloc (the entry point that lays every device buffer out in the library's static scratch array and
allocates nothing) against graph_inference: same plan, same kernels, so the results must be identical bit for bit, on
calls in a row that shrink (stale contents of the shared array must not leak into a later, smaller call).
"""
import numpy as np
import pytest

import ios
from ios.contrib import ios_runtime as rt
from ios.ir import Graph
from oracle import ios_oracle

pytestmark = pytest.mark.gpu


OPTIONS = ('conv_variant', 'conv_split_k', 'autotune', 'executor', 'precision', 'split_k_reduce')


@pytest.fixture(autouse=True)
def closed_form_configurations():
    before = rt.device_info()      # the options in force, put back afterwards whatever the order of the tests
    rt.set_option('conv_variant', -1)
    rt.set_option('conv_split_k', 0)
    rt.set_option('autotune', 0)
    rt.set_option('executor', 'fused')
    rt.set_option('precision', 'fp32')
    rt.set_option('split_k_reduce', 'xcd')
    yield
    for key in OPTIONS:
        value = before[key]
        rt.set_option(key, int(value) if isinstance(value, bool) else value)


def both(graph, batch, seed):
    x = np.random.default_rng(seed).standard_normal((batch, *graph.enter_node.output_shape)).astype(np.float32)
    plain = rt.graph_inference(graph, batch, x)
    static = rt.graph_inference(graph, batch, x, no_alloc=True)
    np.testing.assert_array_equal(static, plain)
    return x, static


def test_the_call_allocates_no_device_memory():
    graph = ios.models.squeezenet_1_1(init_seed=0, init_scheme='he_normal_bias')
    graph.greedy_schedule(4)
    x = np.random.default_rng(0).standard_normal((2, 3, 224, 224)).astype(np.float32)
    rt.device_info()                                   # the device context (streams, address of the static array) exists from here on
    for batch in (2, 1):                               # (and what the HIP runtime sets up by itself on the first launch of a kernel:
        rt.graph_inference(graph, batch, x[:batch], no_alloc=True)   # it loads the code object of a translation unit on first use)
    free = rt.device_free_bytes()
    for batch in (2, 1, 2):
        got = rt.graph_inference(graph, batch, x[:batch], no_alloc=True)
        assert rt.device_free_bytes() == free          # nothing allocated, nothing freed
    np.testing.assert_array_equal(got, rt.graph_inference(graph, 2, x))
    # a session, which owns an allocation, does move the figure (the check above is not vacuous)
    with rt.Session(graph, 2):
        assert rt.device_free_bytes() < free


def test_two_calls_in_a_row_the_second_smaller_equal_graph_inference():
    inception = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    inception.greedy_schedule(8)                       # multi-group stages: the static session still runs them in order
    assert rt.plan_arena_bytes(inception, 1) <= 256 << 20
    x, got = both(inception, 1, seed=1)                # 175 MiB of the 256 MiB array
    err = np.abs(got - ios_oracle.run(inception, x))
    assert (err <= 1e-4 + 1e-3 * np.abs(got)).all()
    squeeze = ios.models.squeezenet_1_1(init_seed=0, init_scheme='he_normal_bias')
    squeeze.sequential_schedule()
    x, got = both(squeeze, 1, seed=2)                  # 21 MiB: runs inside what the first call left behind
    err = np.abs(got - ios_oracle.run(squeeze, x))
    assert (err <= 1e-4 + 1e-3 * np.abs(got)).all()
    both(inception, 1, seed=3)                         # and back


def test_split_k_tickets_and_partial_tiles_live_in_the_static_array():
    ios.reset_name()
    v = ios.placeholder((200, 8, 8))
    block = ios.Block(v.node)
    ios.conv2d(block, [[v]], 136, (3, 3), (1, 1), (1, 1), 1, 'relu', is_exit=True)
    graph = Graph('t', v.node, [block])
    graph.init_weights(seed=5, scheme='he_normal_bias')
    graph.sequential_schedule()
    rt.set_option('conv_split_k', 4)
    for form in ('xcd', 'inline', 'kernel'):
        rt.set_option('split_k_reduce', form)
        for batch in (3, 1, 2, 1):                     # shrinking and growing: tickets must be back at zero every time
            x, got = both(graph, batch, seed=batch)
            err = np.abs(got - ios_oracle.run(graph, x))
            assert (err <= 1e-4 + 1e-3 * np.abs(got)).all()


def test_a_graph_beyond_the_static_array_is_refused_and_the_next_call_works():
    inception = ios.models.inception_v3(init_seed=0, init_scheme='he_normal_bias')
    inception.sequential_schedule()
    assert rt.plan_arena_bytes(inception, 8) <= 256 << 20 < rt.plan_arena_bytes(inception, 12)
    x = np.zeros((12, 3, 299, 299), np.float32)
    with pytest.raises(RuntimeError, match=r'static scratch of graph_inference_no_alloc holds 268435456'):
        rt.graph_inference(inception, 12, x, no_alloc=True)
    sample = ios.models.sample_network(init_seed=0, init_scheme='he_normal_bias')
    sample.sequential_schedule()
    both(sample, 1, seed=4)
    both(sample, 2, seed=4)
