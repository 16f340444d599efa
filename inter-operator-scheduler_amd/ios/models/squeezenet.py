"""
SqueezeNet networks.

``squeezenet_1_1`` is SqueezeNet v1.1 for 3x224x224: conv3x3/2 (64) - maxpool3x3/2 - fire(16,64) x2 -
maxpool - fire(32,128) x2 - maxpool - fire(48,192) x2 - fire(64,256) x2 - conv1x1 (1000) - global average
pool.  A fire module is a 1x1 squeeze convolution followed by parallel 1x1 and 3x3 expand convolutions
whose outputs are concatenated.

``squeezenet`` is the variant the reference ships (python/ios/models/squeezenet.py:4-55): conv7x7/2 (96)
front and fire modules with a residual addition ("complex bypass"), the bypass being the block input or
a 1x1 projection of it.
"""
from .common import Block, Graph, Value, conv2d, identity, placeholder, pool2d, reset_name


def _fire_body(block, v, squeeze, expand):
    s = conv2d(block, [[v]], out_channels=squeeze, kernel=(1, 1))
    e1 = conv2d(block, [[s]], out_channels=expand, kernel=(1, 1))
    e3 = conv2d(block, [[s]], out_channels=expand, kernel=(3, 3), padding=(1, 1))
    return e1, e3


def fire(v: Value, squeeze: int, expand: int):
    block = Block(v.node, None, [], None)
    e1, e3 = _fire_body(block, v, squeeze, expand)
    return identity(block, [[e1], [e3]], is_exit=True), block


def fire_complex(v: Value, squeeze: int, expand: int):
    block = Block(v.node, None, [], None)
    s = conv2d(block, [[v]], out_channels=squeeze, kernel=(1, 1))
    e3 = conv2d(block, [[s]], out_channels=expand, kernel=(3, 3), padding=(1, 1))
    e1 = conv2d(block, [[s]], out_channels=expand, kernel=(1, 1))
    joined = identity(block, [[e3], [e1]])
    if joined.node.output_shape[0] == v.node.output_shape[0]:
        bypass = v
    else:
        bypass = conv2d(block, [[v]], out_channels=2 * expand, kernel=(1, 1))
    return identity(block, [[joined, bypass]], is_exit=True), block


def _maxpool_block(v):
    block = Block(v.node, None, [], None)
    return pool2d(block, [[v]], pool_type='max', kernel=(3, 3), stride=(2, 2), is_exit=True), block


def _classifier_block(v):
    block = Block(v.node, None, [], None)
    v = conv2d(block, [[v]], out_channels=1000, kernel=(1, 1))
    return pool2d(block, [[v]], pool_type='global_avg', is_exit=True), block


def _assemble(name, pv, steps, init_seed, init_scheme):
    blocks = []
    v = pv
    for make, *args in steps:
        v, block = make(v, *args)
        blocks.append(block)
    graph = Graph(name, pv.node, blocks)
    graph.init_weights(init_seed, init_scheme)
    return graph


def squeezenet_1_1(init_seed=None, init_scheme='uniform') -> Graph:
    reset_name()
    pv = placeholder(output_shape=(3, 224, 224))

    def front(v):
        block = Block(v.node, None, [], None)
        v = conv2d(block, [[v]], out_channels=64, kernel=(3, 3), stride=(2, 2))
        return pool2d(block, [[v]], pool_type='max', kernel=(3, 3), stride=(2, 2), is_exit=True), block

    steps = [(front,), (fire, 16, 64), (fire, 16, 64), (_maxpool_block,), (fire, 32, 128), (fire, 32, 128),
             (_maxpool_block,), (fire, 48, 192), (fire, 48, 192), (fire, 64, 256), (fire, 64, 256),
             (_classifier_block,)]
    return _assemble("squeezenet_1_1", pv, steps, init_seed, init_scheme)


def squeezenet(init_seed=None, init_scheme='uniform') -> Graph:
    reset_name()
    pv = placeholder(output_shape=(3, 224, 224))

    def front(v):
        block = Block(v.node, None, [], None)
        v = conv2d(block, [[v]], out_channels=96, kernel=(7, 7), stride=(2, 2), padding=(3, 3))
        return pool2d(block, [[v]], pool_type='max', kernel=(3, 3), stride=(2, 2), is_exit=True), block

    steps = [(front,), (fire_complex, 16, 64), (fire_complex, 16, 64), (fire_complex, 32, 128),
             (_maxpool_block,), (fire_complex, 32, 128), (fire_complex, 48, 192), (fire_complex, 48, 192),
             (fire_complex, 64, 256), (_maxpool_block,), (fire_complex, 64, 256), (_classifier_block,)]
    return _assemble("squeezenet", pv, steps, init_seed, init_scheme)
