"""
Inception-v3 for 3x299x299 inputs without batch norm, auxiliary head and classifier: 13 blocks, 94
convolutions, ends in a global average pool over 2048x8x8.  Topology and operator numbering (names
'0'..'119') follow reference python/ios/models/inception_v3.py:4-128.
"""
from .common import Block, Graph, Value, conv2d, identity, placeholder, pool2d, reset_name


def _chain(block, v, *layers):
    """Apply conv layers given as (out_channels, kernel, padding[, stride]) one after another."""
    for layer in layers:
        out_channels, kernel, padding = layer[:3]
        stride = layer[3] if len(layer) > 3 else (1, 1)
        v = conv2d(block, [[v]], out_channels=out_channels, kernel=kernel, stride=stride, padding=padding)
    return v


def _avg_branch(block, v, out_channels):
    pooled = pool2d(block, [[v]], pool_type='avg', kernel=(3, 3), stride=(1, 1), padding=(1, 1))
    return conv2d(block, [[pooled]], out_channels=out_channels, kernel=(1, 1))


def _concat_exit(block, branches):
    return identity(block, [[b] for b in branches], is_exit=True), block


def inception_front(v: Value):
    # 3x299x299 -> 32x149x149 -> 32x147x147 -> 64x147x147 -> 64x73x73 -> 80x73x73 -> 192x71x71 -> 192x35x35
    block = Block(v.node, None, [], None)
    v = _chain(block, v, (32, (3, 3), (0, 0), (2, 2)), (32, (3, 3), (0, 0)), (64, (3, 3), (1, 1)))
    v = pool2d(block, [[v]], pool_type='max', kernel=(3, 3), stride=(2, 2))
    v = _chain(block, v, (80, (1, 1), (0, 0)), (192, (3, 3), (0, 0)))
    v = pool2d(block, [[v]], pool_type='max', kernel=(3, 3), stride=(2, 2), is_exit=True)
    return v, block


def inception_a(v: Value, pool_features):
    block = Block(v.node, None, [], None)
    b1 = _chain(block, v, (64, (1, 1), (0, 0)))
    b5 = _chain(block, v, (48, (1, 1), (0, 0)), (64, (5, 5), (2, 2)))
    b3 = _chain(block, v, (64, (1, 1), (0, 0)), (96, (3, 3), (1, 1)), (96, (3, 3), (1, 1)))
    bp = _avg_branch(block, v, pool_features)
    return _concat_exit(block, [b1, b5, b3, bp])


def inception_b(v: Value):
    block = Block(v.node, None, [], None)
    b3 = _chain(block, v, (384, (3, 3), (0, 0), (2, 2)))
    bd = _chain(block, v, (64, (1, 1), (0, 0)), (96, (3, 3), (1, 1)), (96, (3, 3), (0, 0), (2, 2)))
    bp = pool2d(block, [[v]], pool_type='max', kernel=(3, 3), stride=(2, 2))
    return _concat_exit(block, [b3, bd, bp])


def inception_c(v: Value, channels_7x7):
    c7 = channels_7x7
    row, col = ((1, 7), (0, 3)), ((7, 1), (3, 0))
    block = Block(v.node, None, [], None)
    b1 = _chain(block, v, (192, (1, 1), (0, 0)))
    b7 = _chain(block, v, (c7, (1, 1), (0, 0)), (c7, *row), (192, *col))
    bd = _chain(block, v, (c7, (1, 1), (0, 0)), (c7, *col), (c7, *row), (c7, *col), (192, *row))
    bp = _avg_branch(block, v, 192)
    return _concat_exit(block, [b1, b7, bd, bp])


def inception_d(v: Value):
    block = Block(v.node, None, [], None)
    b3 = _chain(block, v, (192, (1, 1), (0, 0)), (320, (3, 3), (0, 0), (2, 2)))
    b7 = _chain(block, v, (192, (1, 1), (0, 0)), (192, (1, 7), (0, 3)), (192, (7, 1), (3, 0)),
                (192, (3, 3), (0, 0), (2, 2)))
    bp = pool2d(block, [[v]], pool_type='max', kernel=(3, 3), stride=(2, 2))
    return _concat_exit(block, [b3, b7, bp])


def inception_e(v: Value):
    block = Block(v.node, None, [], None)
    b1 = _chain(block, v, (320, (1, 1), (0, 0)))
    stem3 = _chain(block, v, (384, (1, 1), (0, 0)))
    b3a = _chain(block, stem3, (384, (1, 3), (0, 1)))
    b3b = _chain(block, stem3, (384, (3, 1), (1, 0)))
    stemd = _chain(block, v, (448, (1, 1), (0, 0)), (384, (3, 3), (1, 1)))
    bda = _chain(block, stemd, (384, (1, 3), (0, 1)))
    bdb = _chain(block, stemd, (384, (3, 1), (1, 0)))
    bp = _avg_branch(block, v, 192)
    return _concat_exit(block, [b1, b3a, b3b, bda, bdb, bp])


def inception_logits(v: Value):
    block = Block(v.node, None, [], None)
    v = pool2d(block, [[v]], pool_type='global_avg', is_exit=True)
    return v, block


def inception_v3(init_seed=None, init_scheme='uniform') -> Graph:
    reset_name()
    pv = placeholder(output_shape=(3, 299, 299))
    blocks = []
    v = pv
    recipe = ([(inception_front,)] + [(inception_a, 32), (inception_a, 64), (inception_a, 64)]
              + [(inception_b,)] + [(inception_c, 128), (inception_c, 160), (inception_c, 160),
                                    (inception_c, 192)]
              + [(inception_d,), (inception_e,), (inception_e,), (inception_logits,)])
    for make, *args in recipe:
        v, block = make(v, *args)
        blocks.append(block)
    graph = Graph("inception_v3", pv.node, blocks)
    graph.init_weights(init_seed, init_scheme)
    return graph
