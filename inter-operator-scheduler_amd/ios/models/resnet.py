"""
ResNet-18 / 34 / 50 feature extractors for 3x224x224 (reference python/ios/models/resnet.py:3-83).

Front block: 7x7/2 convolution (64, ReLU) and a 3x3/2 max pooling.  Then four blocks of residual units with 64, 128,
256 and 512 base channels; from the second block on the first unit has stride 2.  A basic unit is 3x3 (ReLU), 3x3
(no activation), plus the skip value, added by an ``element`` operator without an activation after it; a bottleneck
unit is 1x1 (carrying the stride, ReLU), 3x3 (ReLU), 1x1 to four times the base width (no activation), the addition,
and an in-place ReLU.  When the unit changes the shape, the skip value is a 1x1 convolution of the block input with the
unit's stride, which in the reference carries a ReLU (resnet.py:33) and is kept that way.  There is no classifier: the
last residual unit is the exit operator.

The addition of a residual unit and the projection beside the first convolution are what a schedule can run in
parallel here; the networks exercise the two-operand ``element`` operator on the device.
"""
from .common import Block, Graph, activation, addition, conv2d, placeholder, pool2d, reset_name


def _front(v):
    block = Block(v.node, None, [], None)
    v = conv2d(block, [[v]], out_channels=64, kernel=(7, 7), stride=(2, 2), padding=(3, 3), act='relu')
    return pool2d(block, [[v]], pool_type='max', kernel=(3, 3), stride=(2, 2), padding=(1, 1), is_exit=True), block


def _basic_unit(block, v, skip, width, stride, is_exit):
    v = conv2d(block, [[v]], out_channels=width, kernel=(3, 3), stride=stride, padding=(1, 1), act='relu')
    v = conv2d(block, [[v]], out_channels=width, kernel=(3, 3), stride=(1, 1), padding=(1, 1), act='identity')
    return addition(block, [[v, skip]], is_exit=is_exit)


def _bottleneck_unit(block, v, skip, width, stride, is_exit):
    v = conv2d(block, [[v]], out_channels=width, kernel=(1, 1), stride=stride, padding=(0, 0), act='relu')
    v = conv2d(block, [[v]], out_channels=width, kernel=(3, 3), stride=(1, 1), padding=(1, 1), act='relu')
    v = conv2d(block, [[v]], out_channels=4 * width, kernel=(1, 1), stride=(1, 1), padding=(0, 0), act='identity')
    v = addition(block, [[v, skip]])
    return activation(block, [[v]], act_type='relu', inplace=True, is_exit=is_exit)


def _residual_block(v, unit, expansion, width, units, stride):
    block = Block(v.node, None, [], None)
    out_channels = width * expansion
    skip = v
    if max(stride) != 1 or v.node.output_shape[0] != out_channels:
        skip = conv2d(block, [[v]], out_channels=out_channels, kernel=(1, 1), stride=stride, padding=(0, 0), act='relu')
    for i in range(units):
        v = unit(block, v, skip, width, stride if i == 0 else (1, 1), is_exit=i == units - 1)
        skip = v
    return v, block


def _resnet(name, unit, expansion, units_per_block, init_seed, init_scheme) -> Graph:
    reset_name()
    pv = placeholder(output_shape=(3, 224, 224))
    v, front = _front(pv)
    blocks = [front]
    for i, (width, units) in enumerate(zip((64, 128, 256, 512), units_per_block)):
        v, block = _residual_block(v, unit, expansion, width, units, (1, 1) if i == 0 else (2, 2))
        blocks.append(block)
    graph = Graph(name, pv.node, blocks)
    graph.init_weights(init_seed, init_scheme)
    graph.sequential_schedule()
    return graph


def resnet18(init_seed=None, init_scheme='uniform') -> Graph:
    return _resnet('resnet18', _basic_unit, 1, (2, 2, 2, 2), init_seed, init_scheme)


def resnet34(init_seed=None, init_scheme='uniform') -> Graph:
    return _resnet('resnet34', _basic_unit, 1, (3, 4, 6, 3), init_seed, init_scheme)


def resnet50(init_seed=None, init_scheme='uniform') -> Graph:
    return _resnet('resnet50', _bottleneck_unit, 4, (3, 4, 6, 3), init_seed, init_scheme)
