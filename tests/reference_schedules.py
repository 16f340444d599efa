"""
The reference keeps seven optimised Inception-v3 schedules in its wire format (reference
experiments/specialization/schedules/{1,16,32,64,128,k80,v100}.json, read by experiments/specialization/main.py:43-48
through Graph.from_config, python/ios/ir.py:1025-1046).  They are committed unchanged under tests/golden/reference_schedules/
as data fixtures.  This module loads them and gives a loaded graph the weights of the plain model, stacking the weights
of merged convolutions the way the reference's optimizer does (python/ios/optimizer.py:662-711): output channels in
hint-name order, smaller kernels centred inside the common kernel window, zeros around them.
"""
import json
import os

import numpy as np

from ios.ir import Conv, Graph

DIRECTORY = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'reference_schedules')
# file name -> batch size the reference tuned the schedule for (k80 and v100 are batch-1 schedules of two devices)
TUNED_BATCH = {'1': 1, '16': 16, '32': 32, '64': 64, '128': 128, 'k80': 1, 'v100': 1}


def load_config(name):
    with open(os.path.join(DIRECTORY, f'{name}.json')) as f:
        return json.load(f)


def load(name) -> Graph:
    return Graph.from_config(load_config(name))


def adopt_weights(scheduled: Graph, plain: Graph):
    """Weights of ``plain`` (convolutions looked up by name) for every convolution of ``scheduled``."""
    source = {conv.name: conv for conv in plain.conv_nodes()}
    for conv in scheduled.conv_nodes():
        members = [source[token] for token in conv.hint_name.split()]
        assert sum(m.out_channels for m in members) == conv.out_channels
        weight = np.zeros(conv.weight_shape, dtype=np.float32)
        bias = np.zeros(conv.bias_shape, dtype=np.float32)
        first = 0
        for m in members:
            last = first + m.out_channels
            r0, c0 = (conv.kernel[0] - m.kernel[0]) // 2, (conv.kernel[1] - m.kernel[1]) // 2
            assert m.weight.shape[1] == weight.shape[1]
            weight[first:last, :, r0:r0 + m.kernel[0], c0:c0 + m.kernel[1]] = m.weight
            bias[first:last] = m.bias
            first = last
        conv.weight, conv.bias = weight, bias
