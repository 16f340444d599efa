"""
Seeded random networks for the planner and parity tests: small blocks that mix every operator kind the runtime knows
(convolutions with all activations, grouped and depth-wise ones, pools, ReLU / activation nodes, two-operand additions and
products, sums, concatenations, channel slices, separable units, sibling convolutions, residual units) in random wiring,
so that the planner's rewrites (folded ReLUs, concatenations written in place, sums in depth-wise loaders, additions
absorbed by activations or by a convolution's epilogue) meet each other in combinations no hand-written case holds.
"""
import numpy as np

import ios
from ios.ir import Graph, Value


def _pick(rng, items):
    return items[int(rng.integers(len(items)))]


def _maybe_slice(rng, value):
    """The value itself, or a channel slice of it."""
    if value.length >= 4 and rng.random() < 0.25:
        begin = int(rng.integers(0, value.length // 2))
        end = int(rng.integers(begin + 2, value.length + 1))
        return Value(value.node, value.begin + begin, value.begin + end)
    return value


def _same_width(rng, values, like, count):
    """Up to `count` further values with as many channels as `like` (slices of wider ones included)."""
    found = []
    for value in values:
        if value is like or value.length < like.length:
            continue
        begin = 0 if value.length == like.length else int(rng.integers(0, value.length - like.length + 1))
        found.append(Value(value.node, value.begin + begin, value.begin + begin + like.length))
    rng.shuffle(found)
    return found[:count]


def _terms(rng, values, max_terms=2, max_summed=3):
    """A random input: 1..max_terms concatenated terms, each a sum of 1..max_summed values of equal width."""
    terms = []
    for _ in range(int(rng.integers(1, max_terms + 1))):
        first = _maybe_slice(rng, _pick(rng, values))
        term = [first]
        if rng.random() < 0.4:
            term += _same_width(rng, values, first, int(rng.integers(1, max_summed)))
        terms.append(term)
    return terms


def _channels(terms):
    return sum(term[0].length for term in terms)


def random_block(rng, enter, downsample, wide=1):
    block = ios.Block(enter.node)
    values = [enter]
    if downsample:
        if rng.random() < 0.5:
            base = ios.pool2d(block, [[enter]], _pick(rng, ['max', 'avg']), (3, 3), (2, 2), (1, 1))
        else:
            base = ios.conv2d(block, [[enter]], wide * int(rng.integers(4, 17)), (3, 3), (2, 2), (1, 1), 1, _pick(rng, ['relu', 'identity']))
        values = [base]
    for _ in range(int(rng.integers(4, 11))):
        kind = _pick(rng, ['conv', 'conv', 'conv', 'sibling', 'residual', 'depthwise', 'grouped', 'pool', 'relu', 'activation', 'element', 'sum', 'concat', 'separable'])
        if kind == 'conv':
            terms = _terms(rng, values)
            k = _pick(rng, [(1, 1), (1, 1), (3, 3), (3, 3), (1, 3), (3, 1), (5, 5)])
            out = ios.conv2d(block, terms, wide * int(rng.integers(3, 25)), k, (1, 1), (k[0] // 2, k[1] // 2), 1,
                             _pick(rng, ['relu', 'relu', 'identity', 'identity', 'tanh', 'sigmoid']))
        elif kind == 'sibling':
            # a second convolution on the inputs of an earlier one, same stride and activation: what the merge search stacks
            convs = [v.node for v in values if v.node.type == 'conv' and v.node.groups == 1 and v.node.inputs is not None]
            if not convs:
                continue
            twin = _pick(rng, convs)
            k = _pick(rng, [tuple(twin.kernel), (1, 1), (3, 3), (1, 3), (3, 1)])
            out = ios.conv2d(block, [list(term) for term in twin.inputs], wide * int(rng.integers(3, 17)), k, tuple(twin.stride), (k[0] // 2, k[1] // 2), 1, twin.act)
        elif kind == 'residual':
            # convolution, + an earlier value of the same width (, ReLU): what a convolution's epilogue can take over
            skip = _pick(rng, values)
            k = _pick(rng, [(1, 1), (3, 3)])
            y = ios.conv2d(block, _terms(rng, values), skip.length, k, (1, 1), (k[0] // 2, k[1] // 2), 1, _pick(rng, ['identity', 'identity', 'relu']))
            out = ios.addition(block, [[y, skip] if rng.random() < 0.5 else [skip, y]])
            if rng.random() < 0.6:
                out = ios.activation(block, [[out]], _pick(rng, ['relu', 'relu', 'tanh']), bool(rng.integers(2)))
        elif kind == 'depthwise':
            terms = _terms(rng, values, max_terms=1, max_summed=4)
            k = _pick(rng, [3, 3, 5, 7])
            c = _channels(terms)
            out = ios.conv2d(block, terms, c, (k, k), (1, 1), (k // 2, k // 2), c, _pick(rng, ['relu', 'identity']))
        elif kind == 'grouped':
            terms = _terms(rng, values)
            c = _channels(terms)
            groups = 2 if c % 2 == 0 else 1
            out = ios.conv2d(block, terms, groups * wide * int(rng.integers(2, 9)), (3, 3), (1, 1), (1, 1), groups, _pick(rng, ['relu', 'identity']))
        elif kind == 'pool':
            out = ios.pool2d(block, _terms(rng, values, max_terms=1, max_summed=2), _pick(rng, ['max', 'avg']), (3, 3), (1, 1), (1, 1))
        elif kind == 'relu':
            out = ios.relu(block, _terms(rng, values))
        elif kind == 'activation':
            out = ios.activation(block, _terms(rng, values, max_terms=1), _pick(rng, ['relu', 'tanh', 'sigmoid']), bool(rng.integers(2)))
        elif kind == 'element':
            first = _pick(rng, values)
            others = _same_width(rng, values, first, 1)
            if not others:
                continue
            pair = [first, others[0]] if rng.random() < 0.5 else [others[0], first]
            out = ios.addition(block, [pair]) if rng.random() < 0.7 else ios.multiply(block, [pair])
        elif kind == 'sum':
            first = _pick(rng, values)
            others = _same_width(rng, values, first, int(rng.integers(1, 4)))
            if not others:
                continue
            out = ios.identity(block, [[first] + others])
        elif kind == 'concat':
            out = ios.identity(block, _terms(rng, values, max_terms=3))
        else:
            terms = _terms(rng, values, max_terms=1, max_summed=4)
            k = _pick(rng, [3, 5])
            make = ios.relu_sep_conv if rng.random() < 0.7 else ios.sep_conv
            out = make(block, terms, wide * int(rng.integers(4, 17)), (k, k), (1, 1), (k // 2, k // 2))
        values.append(out)
    # the exit concatenates everything nobody has read yet, so that no operator is dead
    loose = [value for value in values[1:] if not value.node.uses] or [values[-1]]
    if len(loose) == 1 and rng.random() < 0.5:
        exit_value = ios.relu(block, [[loose[0]]], is_exit=True)
    else:
        exit_value = ios.identity(block, [[value] for value in loose], is_exit=True)
    return exit_value, block


def random_graph(seed, large=False):
    """
    `large`: eight times the channels on 20-44 pixel sides (several tiles per convolution, long reductions, the wide pooling
    path) instead of 3-24 channels on 5-13 pixel sides.

    (graph with a schedule, batch size, the graph as it was built).  A fifth of the graphs went through the merge search,
    which replaces sibling convolutions by one convolution with stacked filters read through channel slices; the graph as
    built computes the same function and is what a result is checked against.
    """
    rng = np.random.default_rng(seed)
    ios.reset_name()
    wide = 8 if large else 1
    low, high = (20, 45) if large else (5, 14)
    pv = ios.placeholder((wide * int(rng.integers(3, 13)), int(rng.integers(low, high)), int(rng.integers(low, high))))
    value, blocks = pv, []
    for index in range(int(rng.integers(1, 4))):
        value, block = random_block(rng, value, downsample=index > 0 and rng.random() < 0.6, wide=wide)
        blocks.append(block)
    graph = Graph(f'random_{seed}', pv.node, blocks)
    graph.init_weights(seed, 'he_normal_bias')
    built = graph
    batch = int(rng.integers(1, 4))
    choice = int(rng.integers(5))
    if choice == 0:
        graph.sequential_schedule()
    elif choice == 1:
        graph.greedy_schedule(int(rng.integers(2, 9)))
    else:
        graph.sequential_schedule()
        kind = 'dp_parallel' if choice < 4 else _pick(rng, ['dp_merge', 'dp_parallel_merge'])
        graph = ios.optimize(graph, batch, ios.AnalyticCostModel(launch=1.0, rate=float(10 ** rng.integers(4, 8)), sync=float(rng.random())),
                             kind, max_group_size=int(rng.integers(1, 4)), max_num_groups=int(rng.integers(2, 7)), compute_weight=True)
    return graph, batch, built
