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


class IOSCostModel(CostModel):
    """Latency measured by executing on the device (reference cost_model.py:36-48)."""

    def get_graph_latency(self, graph, batch_size, warmup, number, repeat, profile_stage=False):
        from ios.contrib.ios_runtime import graph_latency
        return graph_latency(graph, batch_size, warmup, number, repeat, profile_stage)

    def get_block_latency(self, block, batch_size, warmup, number, repeat, profile_stage=False):
        from ios.contrib.ios_runtime import block_latency
        return block_latency(block, batch_size, warmup, number, repeat, profile_stage)

    def get_stage_latency(self, stage, batch_size, warmup, number, repeat, profile_stage=False):
        from ios.contrib.ios_runtime import stage_latency
        return stage_latency(stage, batch_size, warmup, number, repeat, profile_stage)
