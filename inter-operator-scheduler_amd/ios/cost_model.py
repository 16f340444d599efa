"""
Cost models that price a stage, a block or a graph for the schedule search (interface of reference
python/ios/cost_model.py:7-48).  ``IOSCostModel`` measures on the GPU through the runtime library;
``RandomCostModel`` returns random numbers so that the search can run without a device;
``AnalyticCostModel`` is a deterministic additive model for tests and dry runs.
"""
from typing import List

import numpy as np

from ios.ir import Block, Graph, Node


class CostModel:
    def get_stage_latency(self, stage: List[List[Node]], batch_size, warmup, number, repeat,
                          profile_stage=False) -> List[float]:
        raise NotImplementedError

    def get_block_latency(self, block: Block, batch_size, warmup, number, repeat, profile_stage=False) -> List[float]:
        raise NotImplementedError

    def get_graph_latency(self, graph: Graph, batch_size, warmup, number, repeat, profile_stage=False) -> List[float]:
        raise NotImplementedError


class RandomCostModel(CostModel):
    """Uniform random latencies; pass ``seed`` for reproducible schedules."""

    def __init__(self, seed=None):
        self._rng = np.random if seed is None else np.random.default_rng(seed)

    def _draw(self, repeat):
        return [float(self._rng.random()) for _ in range(repeat)]

    def get_graph_latency(self, graph, batch_size, warmup, number, repeat, profile_stage=False):
        return self._draw(repeat)

    def get_block_latency(self, block, batch_size, warmup, number, repeat, profile_stage=False):
        return self._draw(repeat)

    def get_stage_latency(self, stage, batch_size, warmup, number, repeat, profile_stage=False):
        return self._draw(repeat)


class AnalyticCostModel(CostModel):
    """
    Deterministic model: an operator costs ``launch + flops / rate``; a group costs the sum of its
    operators; a stage costs the longest group plus ``sync`` per additional group.  Units are arbitrary.
    """

    def __init__(self, launch=1.0, rate=1e6, sync=0.25):
        self.launch, self.rate, self.sync = launch, rate, sync

    def op_cost(self, node: Node, batch_size):
        return self.launch * max(1, node.kernels()) + batch_size * node.flops() / self.rate

    def get_stage_latency(self, stage, batch_size, warmup, number, repeat, profile_stage=False):
        longest = max(sum(self.op_cost(node, batch_size) for node in group) for group in stage)
        return [longest + self.sync * (len(stage) - 1)] * repeat

    def get_block_latency(self, block, batch_size, warmup, number, repeat, profile_stage=False):
        by_name = {node.name: node for node in block.inner_nodes + [block.exit_node]}
        total = sum(self.get_stage_latency([[by_name[n] for n in group] for group in stage], batch_size,
                                           warmup, number, 1)[0] for stage in block.stages)
        return [total] * repeat

    def get_graph_latency(self, graph, batch_size, warmup, number, repeat, profile_stage=False):
        total = sum(self.get_block_latency(block, batch_size, warmup, number, 1)[0] for block in graph.blocks)
        return [total] * repeat


def stage_signature(stage: List[List[Node]]) -> str:
    """
    The stage's two runtime documents with every operator name replaced by its position of first appearance: two stages
    with the same signature are the same computation on tensors of the same shapes (the repeated cells of NASNet, the
    equal-width blocks of Inception-v3), whatever their operators are called.
    """
    from ios.contrib.ios_runtime import stage_documents
    import json
    stage_json, input_json = stage_documents(stage)
    groups, producers = json.loads(stage_json), json.loads(input_json)
    order = {}

    def number(name):
        return order.setdefault(name, len(order))

    def declare(config):
        number(config['name'])
        for child in config.get('nodes', []):
            declare(child)

    def rewrite(config):
        out = {key: value for key, value in config.items() if key not in ('name', 'hint_name', 'inputs', 'nodes')}
        out['name'] = number(config['name'])
        if config.get('inputs') is not None:
            out['inputs'] = [[[number(producer), begin, end] for producer, begin, end in term] for term in config['inputs']]
        if 'nodes' in config:
            out['nodes'] = [rewrite(child) for child in config['nodes']]
        return out

    for group in groups:
        for config in group:
            declare(config)
    body = [[rewrite(config) for config in group] for group in groups]
    outside = sorted((number(name), shape) for name, shape in producers.items())
    return json.dumps([body, outside], sort_keys=True)


class IOSCostModel(CostModel):
    """
    Latency measured by executing on the device (reference cost_model.py:36-48).

    ``share_identical_stages=True`` measures stages that are the same computation on the same shapes once per model
    instance (see ``stage_signature``) and returns that measurement for all of them: the search over a network of
    repeated cells asks for far fewer measurements and identical cells get identical schedules.  The measurements depend
    on the runtime options in force (executor, precision, ...): use a new instance after changing them.  Off by default,
    like the reference, where every request is a measurement.
    """

    def __init__(self, share_identical_stages=False):
        self.share_identical_stages = share_identical_stages
        self.measured_stages = 0
        self._by_signature = {}

    def get_graph_latency(self, graph, batch_size, warmup, number, repeat, profile_stage=False):
        from ios.contrib.ios_runtime import graph_latency
        return graph_latency(graph, batch_size, warmup, number, repeat, profile_stage)

    def get_block_latency(self, block, batch_size, warmup, number, repeat, profile_stage=False):
        from ios.contrib.ios_runtime import block_latency
        return block_latency(block, batch_size, warmup, number, repeat, profile_stage)

    def get_stage_latency(self, stage, batch_size, warmup, number, repeat, profile_stage=False):
        if not self.share_identical_stages:
            self.measured_stages += 1
            return self._measure_stage(stage, batch_size, warmup, number, repeat, profile_stage)
        key = (stage_signature(stage), batch_size, warmup, number, repeat, bool(profile_stage))
        if key not in self._by_signature:
            self.measured_stages += 1
            self._by_signature[key] = self._measure_stage(stage, batch_size, warmup, number, repeat, profile_stage)
        found = self._by_signature[key]
        return (list(found[0]), list(found[1])) if isinstance(found, tuple) else list(found)

    @staticmethod
    def _measure_stage(stage, batch_size, warmup, number, repeat, profile_stage):
        from ios.contrib.ios_runtime import stage_latency
        return stage_latency(stage, batch_size, warmup, number, repeat, profile_stage)
