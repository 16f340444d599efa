"""
Builder functions that append operators to a block (API of reference python/ios/models/common.py:12-516).

Every function creates the operator, infers its shape, records it in the ``uses`` list of its producers
and stores it either as an inner operator or as the exit operator of ``block``.  The returned ``Value``
covers all output channels of the new operator.  Operator names are consecutive decimal strings taken
from a module-wide counter; call ``reset_name()`` before building a new network.
"""
from typing import List, Tuple

from ios.ir import (Activation, Block, Conv, Element, Graph, Identity, Node, Placeholder, Pool, Relu,
                    Sequential, Value)

_next_index = 0


def new_name():
    global _next_index
    name = str(_next_index)
    _next_index += 1
    return name


def reset_name():
    global _next_index
    _next_index = 0


def _attach(block: Block, node: Node, is_exit: bool) -> Value:
    node.infer_shape()
    node._register_uses()
    if is_exit:
        block.exit_node = node
    else:
        block.inner_nodes.append(node)
    return Value(node, 0, node.output_shape[0])


def placeholder(output_shape):
    name = new_name()
    holder = Placeholder(name, name, output_shape)
    return Value(holder, 0, output_shape[0])


def conv2d(block: Block, inputs, out_channels, kernel=(1, 1), stride=(1, 1), padding=(0, 0), groups=1,
           act="relu", is_exit=False):
    name = new_name()
    return _attach(block, Conv(name, name, inputs, out_channels, kernel, stride, padding, groups, act,
                               None), is_exit)


def pool2d(block: Block, inputs, pool_type, kernel=(1, 1), stride=(1, 1), padding=(0, 0), is_exit=False):
    name = new_name()
    return _attach(block, Pool(name, name, inputs, pool_type, kernel, stride, padding, None), is_exit)


def identity(block: Block, inputs, is_exit=False):
    name = new_name()
    return _attach(block, Identity(name, name, inputs, None), is_exit)


def relu(block: Block, inputs, is_exit=False):
    name = new_name()
    return _attach(block, Relu(name, name, inputs, None), is_exit)


def activation(block: Block, inputs, act_type, inplace, is_exit=False):
    name = new_name()
    return _attach(block, Activation(name, name, inputs, act_type=act_type, inplace=inplace,
                                     output_shape=None), is_exit)


def sigmoid(block: Block, inputs, inplace=False, is_exit=False):
    return activation(block, inputs, 'sigmoid', inplace, is_exit)


def tanh(block: Block, inputs, inplace=False, is_exit=False):
    return activation(block, inputs, 'tanh', inplace, is_exit)


def element(block: Block, inputs, op_type, is_exit=False):
    name = new_name()
    return _attach(block, Element(name, name, inputs, op_type=op_type, output_shape=None), is_exit)


def multiply(block: Block, inputs, is_exit=False):
    return element(block, inputs, op_type='mul', is_exit=is_exit)


def addition(block: Block, inputs, is_exit=False):
    return element(block, inputs, op_type='add', is_exit=is_exit)


def sequential(block: Block, hint_name, nodes: List[Node], is_exit=False):
    """
    Chain ``nodes`` into one schedule unit: ``nodes[0]`` keeps its inputs, every later node reads the
    whole output of its predecessor (reference common.py:327-362).
    """
    name = new_name()
    for prev, cur in zip(nodes, nodes[1:]):
        prev.infer_shape()
        cur.inputs = [[Value(prev, 0, prev.output_shape[0])]]
    return _attach(block, Sequential(name, name if hint_name is None else hint_name, nodes, None), is_exit)


def _pointwise_conv(out_channels):
    name = new_name()
    return Conv(name, name, None, out_channels=out_channels, kernel=(1, 1), stride=(1, 1),
                padding=(0, 0), groups=1, act="identity", output_shape=None)


def _depthwise_conv(inputs, channels, kernel, stride, padding):
    name = new_name()
    return Conv(name, name, inputs, out_channels=channels, kernel=kernel, stride=stride,
                padding=padding, groups=channels, act="identity", output_shape=None)


def _channels_of(inputs):
    # channels of the concatenated terms; a term's width is that of its values, which may be channel slices (the reference
    # takes the producer's full width here, python/ios/models/common.py:396,436, and builds an invalid depth-wise convolution
    # from a sliced input; for whole values the two agree)
    return sum(term[0].end - term[0].begin for term in inputs)


def sep_conv(block: Block, inputs: List[List[Value]], out_channels, kernel, stride, padding, is_exit=False):
    """Depth-wise convolution followed by a 1x1 convolution, no activations."""
    depthwise = _depthwise_conv(inputs, _channels_of(inputs), kernel, stride, padding)
    pointwise = _pointwise_conv(out_channels)
    return sequential(block, 'SepConv', [depthwise, pointwise], is_exit)


def relu_sep_conv(block: Block, inputs: List[List[Value]], out_channels, kernel, stride, padding,
                  is_exit=False):
    """ReLU, depth-wise convolution, 1x1 convolution."""
    name = new_name()
    front = Relu(name, name, inputs, None)
    depthwise = _depthwise_conv(None, _channels_of(inputs), kernel, stride, padding)
    pointwise = _pointwise_conv(out_channels)
    return sequential(block, 'ReluSepConv', [front, depthwise, pointwise], is_exit)


def relu_conv(block: Block, inputs, out_channels, kernel=(1, 1), stride=(1, 1), padding=(0, 0), groups=1,
              is_exit=False):
    """ReLU followed by a convolution without activation."""
    relu_name, conv_name = new_name(), new_name()
    nodes = [Relu(relu_name, relu_name, inputs, None),
             Conv(conv_name, conv_name, None, out_channels=out_channels, kernel=kernel, stride=stride,
                  padding=padding, groups=groups, act="identity", output_shape=None)]
    return sequential(block, 'ReluConv', nodes, is_exit)


def rwconv2d(block: Block, inputs, out_channels, stride=(1, 1), is_exit=False):
    """RandWire node operator: ReLU + separable 3x3 convolution with padding 1."""
    return relu_sep_conv(block, inputs, out_channels, (3, 3), stride, (1, 1), is_exit)


def get_parts(block, split_vars: List[Value]):
    """
    Partition the operators of a large block for the schedule search: part i holds the operators whose
    numeric name lies in (split_vars[i], split_vars[i + 1]] (reference common.py:486-516).
    """
    bounds = [int(v.node.name) for v in split_vars]
    parts = [[] for _ in range(len(bounds) - 1)]
    for node in block.inner_nodes + [block.exit_node]:
        index = int(node.name)
        slot = next((i for i in range(len(bounds) - 1) if bounds[i] < index <= bounds[i + 1]), None)
        assert slot is not None, f'operator {node.name} lies outside the split points {bounds}'
        parts[slot].append(node)
    return parts
