"""
The AlexNet feature extractor of the reference's model zoo (python/ios/models/alexnet.py:4-21) for 3x224x224: 11x11/4
convolution (64), 3x3/2 max pooling, 5x5 convolution (192), 3x3/2 max pooling, then three 3x3 convolutions without
padding (384, 256, 256), all with ReLU, in a single block; the last convolution is the exit operator.  The reference
spells the pooling type 'max_pool'; its runtime only looks for the substring "max" (src/ios/ios_runtime.cu:1047-1050),
so the canonical 'max' used here means the same operator.
"""
from .common import Block, Graph, conv2d, placeholder, pool2d, reset_name


def alexnet(init_seed=None, init_scheme='uniform') -> Graph:
    reset_name()
    pv = placeholder(output_shape=(3, 224, 224))
    block = Block(pv.node, None, [], None)
    v = conv2d(block, [[pv]], out_channels=64, kernel=(11, 11), stride=(4, 4), padding=(2, 2))
    v = pool2d(block, [[v]], pool_type='max', kernel=(3, 3), stride=(2, 2), padding=(1, 1))
    v = conv2d(block, [[v]], out_channels=192, kernel=(5, 5), stride=(1, 1), padding=(2, 2))
    v = pool2d(block, [[v]], pool_type='max', kernel=(3, 3), stride=(2, 2), padding=(1, 1))
    for i, width in enumerate((384, 256, 256)):
        v = conv2d(block, [[v]], out_channels=width, kernel=(3, 3), stride=(1, 1), padding=(0, 0), is_exit=i == 2)
    graph = Graph('alexnet', pv.node, [block])
    graph.init_weights(init_seed, init_scheme)
    graph.sequential_schedule()
    return graph
