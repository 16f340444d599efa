"""
VGG-11 / 13 / 16 / 19 feature extractors for 3x224x224 (reference python/ios/models/vgg.py:3-42): one block of 3x3
convolutions (padding 1, ReLU) in five groups of 64 / 128 / 256 / 512 / 512 channels, a 2x2 max pooling of stride 2
after every group, and a global average pooling as the exit operator.  The networks are chains: they have no
inter-operator parallelism and serve as the sequential end of the model zoo.
"""
from .common import Block, Graph, conv2d, placeholder, pool2d, reset_name

# convolutions per group (64, 128, 256, 512, 512 channels)
_DEPTHS = {'vgg_11': (1, 1, 2, 2, 2), 'vgg_13': (2, 2, 2, 2, 2), 'vgg_16': (2, 2, 3, 3, 3), 'vgg_19': (2, 2, 4, 4, 4)}
_WIDTHS = (64, 128, 256, 512, 512)


def _vgg(name, init_seed, init_scheme) -> Graph:
    reset_name()
    pv = placeholder(output_shape=(3, 224, 224))
    block = Block(pv.node, None, [], None)
    v = pv
    for width, depth in zip(_WIDTHS, _DEPTHS[name]):
        for _ in range(depth):
            v = conv2d(block, [[v]], out_channels=width, kernel=(3, 3), stride=(1, 1), padding=(1, 1), act='relu')
        v = pool2d(block, [[v]], pool_type='max', kernel=(2, 2), stride=(2, 2))
    pool2d(block, [[v]], pool_type='global_avg', is_exit=True)
    graph = Graph(name, pv.node, [block])
    graph.init_weights(init_seed, init_scheme)
    graph.sequential_schedule()
    return graph


def vgg_11(init_seed=None, init_scheme='uniform') -> Graph:
    return _vgg('vgg_11', init_seed, init_scheme)


def vgg_13(init_seed=None, init_scheme='uniform') -> Graph:
    return _vgg('vgg_13', init_seed, init_scheme)


def vgg_16(init_seed=None, init_scheme='uniform') -> Graph:
    return _vgg('vgg_16', init_seed, init_scheme)


def vgg_19(init_seed=None, init_scheme='uniform') -> Graph:
    return _vgg('vgg_19', init_seed, init_scheme)
