"""
The four-convolution demonstration network of the reference README (README.md:103-113,
examples/sample.py:5-15): 375x15x15 input, three 3x3 branches, one of them two convolutions deep,
concatenated to 1875x15x15.
"""
from .common import Block, Graph, conv2d, identity, placeholder, reset_name


def sample_network(init_seed=None, init_scheme='uniform') -> Graph:
    reset_name()
    v = placeholder(output_shape=(375, 15, 15))
    block = Block(enter_node=v.node)
    args = dict(kernel=(3, 3), stride=(1, 1), padding=(1, 1), act='relu')
    v1 = conv2d(block, inputs=[[v]], out_channels=375, **args)
    v2 = conv2d(block, inputs=[[v]], out_channels=750, **args)
    v3 = conv2d(block, inputs=[[v]], out_channels=375, **args)
    v1 = conv2d(block, inputs=[[v1]], out_channels=750, **args)
    identity(block, inputs=[[v1], [v2], [v3]], is_exit=True)
    graph = Graph(name="demo", input=v.node, blocks=[block])
    graph.init_weights(init_seed, init_scheme)
    return graph
