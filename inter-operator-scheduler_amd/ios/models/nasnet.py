"""
NASNet-A networks built as one large block that is split into per-cell parts for the schedule search.

Cell wiring follows reference python/ios/models/nasnet.py:26-135 (stem0, stem1, first cell, normal
cell, reduction cell: five branches per cell, each branch the sum of two operators drawn from separable
3x3/5x5/7x7 convolutions, 3x3 average/max pooling and identity; the branch outputs are concatenated).
The reference hard-wires NASNet-A large (6 cells per stack, 331x331 input, :138-177); here the number of
cells per stack, the filter counts and the input size are parameters, ``nasnet_mobile`` is 4 @ 1056 on
224x224 and ``nasnet_large`` is 6 @ 4032 on 331x331.
"""
from .common import (Block, Graph, Value, conv2d, get_parts, identity, placeholder, pool2d, relu,
                     relu_conv, relu_sep_conv, reset_name)


def _sep(block, x: Value, out_channels, k, stride, keep_width=True) -> Value:
    """Two stacked ReLU-separable convolutions; the first keeps (or directly sets) the channel count."""
    mid = x.node.output_shape[0] if keep_width else out_channels
    pad = (k // 2, k // 2)
    x = relu_sep_conv(block, [[x]], mid, (k, k), (stride, stride), pad)
    return relu_sep_conv(block, [[x]], out_channels, (k, k), (1, 1), pad)


def _pool(block, x: Value, kind, stride) -> Value:
    return pool2d(block, [[x]], pool_type=kind, kernel=(3, 3), stride=(stride, stride), padding=(1, 1))


def _proj(block, x: Value, out_channels, stride=1) -> Value:
    return relu_conv(block, [[x]], out_channels, kernel=(1, 1), stride=(stride, stride), padding=(0, 0))


def _reduction_body(block, pooled: Value, convolved: Value, width, stem_style):
    """
    Shared wiring of stem0 / stem1 / reduction cell.  ``pooled`` feeds the three strided poolings and
    the 5x5 half of branch 0, ``convolved`` feeds the 7x7, 7x7 and 5x5 separable halves.
    """
    keep = not stem_style
    c0 = identity(block, [[_sep(block, pooled, width, 5, 2), _sep(block, convolved, width, 7, 2, keep)]])
    c1l = _pool(block, pooled, 'max', 2)
    c1r = _sep(block, convolved, width, 7, 2, keep)
    c1 = identity(block, [[c1l, c1r]])
    c2l = _pool(block, pooled, 'avg', 2)
    c2r = _sep(block, convolved, width, 5, 2, keep)
    c3r = _pool(block, c0, 'avg', 1)
    c4l = _sep(block, c0, width, 3, 1)
    c4r = _pool(block, pooled, 'max', 2)
    return c0, c1l, c1r, c1, c2l, c2r, c3r, c4l, c4r


def stem0(block, x: Value, num_filters) -> Value:
    x1 = _proj(block, x, num_filters)
    c0, _, _, c1, c2l, c2r, c3r, c4l, c4r = _reduction_body(block, x1, x, num_filters, True)
    return identity(block, [[c1], [c2l, c2r], [c3r, c0], [c4l, c4r]])


def stem1(block, hp: Value, h: Value, num_filters) -> Value:
    x_left = _proj(block, hp, num_filters)
    halves = [_proj(block, h, num_filters // 2, stride=2) for _ in range(2)]
    x_right = identity(block, [halves])
    _, _, _, c1, c2l, c2r, c3r, c4l, c4r = _reduction_body(block, x_left, x_right, num_filters, False)
    return identity(block, [[c1], [c2l, c2r], [c3r, c1], [c4l, c4r]])


def reduction_cell(block, x: Value, x_prev: Value, out_channels_left, out_channels_right) -> Value:
    x_left = _proj(block, x_prev, out_channels_left)
    x_right = _proj(block, x, out_channels_right)
    _, c1l, c1r, c1, c2l, c2r, c3r, c4l, c4r = _reduction_body(block, x_right, x_left, out_channels_right,
                                                               False)
    return identity(block, [[c1l, c1r], [c2l, c2r], [c1, c3r], [c4l, c4r]])


def _normal_body(block, x_left: Value, x_right: Value, width_left, width_right, c0r_from_right):
    """The five summed branch pairs shared by the first cell and the normal cell."""
    c0l = _sep(block, x_right, width_right, 5, 1)
    c0r = _sep(block, x_right, width_right, 3, 1) if c0r_from_right else _sep(block, x_left, width_left, 3, 1)
    c1l = _sep(block, x_left, width_left, 5, 1)
    c1r = _sep(block, x_left, width_left, 3, 1)
    c2l = _pool(block, x_right, 'avg', 1)
    c3l = _pool(block, x_left, 'avg', 1)
    c3r = _pool(block, x_left, 'avg', 1)
    c4l = _sep(block, x_right, width_right, 3, 1)
    return [[c0l, c0r], [c1l, c1r], [c2l, x_left], [c3l, c3r], [c4l, x_right]]


def first_cell(block, x: Value, x_prev: Value, out_channels_left, out_channels_right) -> Value:
    halves = [_proj(block, x_prev, out_channels_left, stride=2) for _ in range(2)]
    x_left = identity(block, [[halves[0]], [halves[1]]])
    x_right = _proj(block, x, out_channels_right)
    terms = _normal_body(block, x_left, x_right, out_channels_right, out_channels_right, True)
    return identity(block, [[x_left]] + terms)


def normal_cell(block, x: Value, x_prev: Value, out_channels_left, out_channels_right) -> Value:
    x_left = _proj(block, x_prev, out_channels_left)
    x_right = _proj(block, x, out_channels_right)
    return identity(block, _normal_body(block, x_left, x_right, out_channels_left, out_channels_right, False))


def nasnet(name, input_size, stem_filters, filters, cells_per_stack, init_seed=None, init_scheme='uniform') -> Graph:
    """
    NASNet-A with ``cells_per_stack`` cells (one first cell + normal cells) in each of the three stacks
    and ``filters`` channels per branch in the first stack; the final feature map has 20*filters channels (the
    reference's normal cell concatenates five sums, python/ios/models/nasnet.py:112, where the published cell also
    passes one of its inputs through: 880 instead of 1056 channels for the mobile model, 3360 instead of 4032 for the large one).
    Every cell output is a split point of ``block.parts``.
    """
    reset_name()
    v0 = placeholder(output_shape=(3, input_size, input_size))
    block = Block(v0.node, None, [], None)
    v1 = conv2d(block, [[v0]], out_channels=stem_filters, kernel=(3, 3), stride=(2, 2), padding=(0, 0),
                act="identity")
    v2 = stem0(block, v1, filters // 4)
    v3 = stem1(block, v2, v1, filters // 2)
    cells = [v2, v3]
    for stack in range(3):
        width = filters << stack
        if stack > 0:
            # the first cell after a reduction down-samples the reduction cell's "previous" input itself
            before = cells[-2]
            cells.append(reduction_cell(block, cells[-1], before, width, width))
            cells.append(first_cell(block, cells[-1], before, width // 2, width))
        else:
            cells.append(first_cell(block, cells[-1], cells[-2], width // 2, width))
        for _ in range(cells_per_stack - 1):
            cells.append(normal_cell(block, cells[-1], cells[-2], width, width))
    tail = relu(block, [[cells[-1]]])
    last = pool2d(block, [[tail]], pool_type='global_avg', is_exit=True)
    block.parts = get_parts(block, split_vars=[v0, v1] + cells + [tail, last])
    graph = Graph(name, v0.node, [block])
    graph.init_weights(init_seed, init_scheme)
    return graph


def nasnet_mobile(init_seed=None, init_scheme='uniform') -> Graph:
    """NASNet-A mobile, 4 @ 1056, 3x224x224 input."""
    return nasnet("nasnet_mobile", 224, 32, 44, 4, init_seed, init_scheme)


def nasnet_large(stem_filters=96, filters=168, init_seed=None, init_scheme='uniform') -> Graph:
    """NASNet-A large, 6 @ 4032, 3x331x331 input (parameters of reference python/ios/models/nasnet.py:138)."""
    return nasnet("nasnet_large", 331, stem_filters, filters, 6, init_seed, init_scheme)
