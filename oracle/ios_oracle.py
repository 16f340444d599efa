"""
CPU oracle for the operator and graph semantics of the inter-operator scheduler runtime.

TEST INFRASTRUCTURE ONLY: this module is the checker used by tests, by the smoke entry point and by the
CPU-baseline leg of the benchmark.  Nothing in the shipped runtime imports it.

It evaluates an exported graph document (the JSON wire format, reference python/ios/ir.py:1038-1046) in
float32 with torch-CPU tensor routines used as a library.  Semantics restated from the reference:

* input algebra (reference python/ios/torch_utils.py:75-125, src/ios/ios_runtime.cu:623-812): every
  operator input is concat_C over terms of sum over values of channel slice [begin, end); an ``element``
  operator with op_type 'mul' multiplies the values of its term instead.
* conv (torch_utils.py:8-26; ios_runtime.cu:254-255,275-277): cross-correlation, zero padding, stride,
  groups, bias, then relu / tanh / sigmoid / identity; output size 1 + (H - KH + 2p) // s.
* pool (torch_utils.py:27-35; ios_runtime.cu:542-550,1047-1057): 'max' ignores padding; 'avg' divides
  by KH*KW including padded positions; a type containing 'global' pools the whole map to 1x1; a type
  containing 'max' is a max pool, everything else an average pool.
* relu / activation / identity / sequential (torch_utils.py:36-57; ios_runtime.cu:912-1035).
* schedule: ``stages`` never change results; the oracle evaluates operators in definition order.

Pinning of this oracle (see tests/test_oracle.py): every torch routine used here is checked against
``brute.py`` (explicit Python loops written from the formulas above) on small shapes including padded
borders, strides, groups and asymmetric kernels, against the plain-C restatement ``conv_ref.c`` on medium
shapes, and against closed forms (1x1 convolution == matrix product, delta kernel == shift, linearity,
block-diagonal equivalence of grouped convolution, global average == mean).  The reference holds no
golden vectors for this path.
"""
from typing import Dict, Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F

Weights = Dict[str, Tuple[np.ndarray, np.ndarray]]

_ACTS = {
    'identity': lambda t: t,
    'relu': torch.relu,
    'tanh': torch.tanh,
    'sigmoid': torch.sigmoid,
}


def conv2d(x, weight, bias, stride, padding, groups, act):
    y = F.conv2d(x, weight, bias, stride=tuple(stride), padding=tuple(padding), groups=groups)
    return _ACTS[act](y)


def pool2d(x, pool_type, kernel, stride, padding):
    if 'global' in pool_type:
        kernel, stride, padding = tuple(x.shape[2:]), (1, 1), (0, 0)
    if 'max' in pool_type:
        return F.max_pool2d(x, tuple(kernel), tuple(stride), tuple(padding))
    return F.avg_pool2d(x, tuple(kernel), tuple(stride), tuple(padding), count_include_pad=True)


def gather_input(inputs, outputs, multiply=False):
    """Evaluate the input algebra: slice, combine the values of each term, concatenate the terms."""
    terms = []
    for term in inputs:
        acc = None
        for name, begin, end in term:
            piece = outputs[name][:, begin:end]
            if acc is None:
                acc = piece
            else:
                acc = acc * piece if multiply else acc + piece
        terms.append(acc)
    return terms[0] if len(terms) == 1 else torch.cat(terms, dim=1)


def to_bf16(t):
    """Round to bfloat16 (nearest even) and back: the reduced-precision mode's view of a convolution operand."""
    return t.to(torch.bfloat16).to(torch.float32)


def to_fp16(t):
    """Round to IEEE half (nearest even, overflow to infinity) and back: the operand view of the precision=fp16 mode."""
    return t.to(torch.float16).to(torch.float32)


def eval_node(config, outputs, weights: Weights, bf16_convs=frozenset(), fp16_convs=frozenset()):
    kind = config['type']
    if kind == 'sequential':
        out = None
        for child in config['nodes']:
            out = eval_node(child, outputs, weights, bf16_convs, fp16_convs)
            outputs[child['name']] = out
        return out
    x = gather_input(config['inputs'], outputs, multiply=(kind == 'element' and config['op_type'] == 'mul'))
    if kind == 'conv':
        w, b = weights[config['name']]
        w = torch.from_numpy(np.ascontiguousarray(w, dtype=np.float32))
        if config['name'] in bf16_convs:   # bfloat16 operands, fp32 accumulation
            x, w = to_bf16(x), to_bf16(w)
        elif config['name'] in fp16_convs:   # half operands, fp32 accumulation
            x, w = to_fp16(x), to_fp16(w)
        return conv2d(x, w,
                      torch.from_numpy(np.ascontiguousarray(b, dtype=np.float32)),
                      config['stride'], config['padding'], config['groups'], config['act'])
    if kind == 'pool':
        return pool2d(x, config['pool_type'], config['kernel'], config['stride'], config['padding'])
    if kind in ('identity', 'element'):
        return x
    if kind == 'relu':
        return torch.relu(x)
    if kind == 'activation':
        return _ACTS[config['act_type']](x)
    raise ValueError(f'unrecognized node type {kind}')


def run_graph(graph_config: dict, weights: Weights, x: np.ndarray, keep_all=False, num_threads: Optional[int] = None,
              bf16_convs=frozenset(), fp16_convs=frozenset()):
    """
    Evaluate an exported graph on input ``x`` (batch, C, H, W).  Returns the exit operator's output as a
    float32 array, or a dict name -> array of every operator when ``keep_all``.  Convolutions named in
    ``bf16_convs`` / ``fp16_convs`` see their input and filters rounded to bfloat16 / IEEE half (the runtime's
    reduced-precision modes).
    """
    if num_threads is not None:
        torch.set_num_threads(num_threads)
    outputs = {graph_config['input']['name']: torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32))}
    last = None
    with torch.no_grad():
        for block in graph_config['blocks']:
            for config in block['inner_nodes'] + [block['exit_node']]:
                outputs[config['name']] = eval_node(config, outputs, weights, bf16_convs, fp16_convs)
                last = config['name']
    if keep_all:
        return {name: t.numpy() for name, t in outputs.items()}
    return outputs[last].numpy()


def graph_weights(graph) -> Weights:
    """name -> (weight, bias) of every convolution of an ``ios.Graph`` (including nested ones)."""
    return {conv.name: (conv.weight, conv.bias) for conv in graph.conv_nodes()}


def run(graph, x: np.ndarray, keep_all=False, num_threads=None, bf16_convs=frozenset(), fp16_convs=frozenset()):
    """Evaluate an ``ios.Graph`` object with the weights stored in its convolutions."""
    return run_graph(graph.export_config(), graph_weights(graph), x, keep_all, num_threads, bf16_convs, fp16_convs)
