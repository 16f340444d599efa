"""
RandWire networks: stages whose wiring is a random Watts-Strogatz graph turned into a DAG by directing
every edge from the lower to the higher node index.

Stage semantics follow reference python/ios/models/randwire.py:44-69: every graph node is a
ReLU + separable 3x3 convolution unit whose input is the sum of its predecessors; nodes without
predecessors read the stage input with stride 2; the stage output is the sum of all nodes without
successors.  The reference reads fixed edge lists from files (:8-17) produced by an unseeded
generator; here ``watts_strogatz_edges`` generates them from a seed and ``read_graph`` still accepts the
file format (line 1: n, line 2: m, then m lines "u v" with u < v).

``randwire_small`` is the configuration with three stages of 32 nodes (k=4, p=0.75) and 78/156/312
channels behind the two-convolution small front.  ``randwire_large`` (:72-87) and ``randwire_xlarge``
(:89-101) are the reference's models; their graphs come from the seeded generator with the reference's
parameters, or from edge-list files in the reference's format (``graph_files`` / ``graph_file``).
"""
from typing import List, Sequence, Tuple

import numpy as np

from .common import (Block, Graph, Value, conv2d, identity, placeholder, pool2d, relu, reset_name,
                     rwconv2d)

Edges = List[Tuple[int, int]]


def watts_strogatz_edges(n: int, k: int, p: float, seed: int) -> Edges:
    """
    Watts-Strogatz small-world graph: ring of ``n`` nodes each joined to its ``k`` nearest neighbours,
    then every edge (i, i+j), j = 1..k/2, is rewired with probability ``p`` to a uniformly chosen node that
    is neither ``i`` nor already adjacent to ``i``.  Returns the sorted undirected edge list as (u, v), u < v.
    """
    assert k % 2 == 0 and 0 < k < n
    rng = np.random.default_rng(seed)
    adjacent = [set() for _ in range(n)]
    for i in range(n):
        for j in range(1, k // 2 + 1):
            adjacent[i].add((i + j) % n)
            adjacent[(i + j) % n].add(i)
    for j in range(1, k // 2 + 1):
        for i in range(n):
            if rng.random() >= p:
                continue
            old = (i + j) % n
            if old not in adjacent[i]:
                continue
            free = [x for x in range(n) if x != i and x not in adjacent[i]]
            if not free:
                continue
            new = free[int(rng.integers(len(free)))]
            adjacent[i].discard(old)
            adjacent[old].discard(i)
            adjacent[i].add(new)
            adjacent[new].add(i)
    return sorted((u, v) for u in range(n) for v in adjacent[u] if u < v)


def read_graph(fname) -> Tuple[int, Edges]:
    with open(fname, 'r') as f:
        tokens = f.read().split()
    n, m = int(tokens[0]), int(tokens[1])
    pairs = tokens[2:2 + 2 * m]
    return n, [(int(pairs[2 * i]), int(pairs[2 * i + 1])) for i in range(m)]


def write_graph(fname, n: int, edges: Edges):
    with open(fname, 'w') as f:
        f.write(f'{n}\n{len(edges)}\n')
        for u, v in edges:
            f.write(f'{u} {v}\n')


def randwire_small_front(v: Value, ch: int):
    block = Block(v.node, None, [], None)
    v = conv2d(block, [[v]], out_channels=ch // 2, kernel=(3, 3), stride=(2, 2), padding=(1, 1), act="relu")
    v = conv2d(block, [[v]], out_channels=ch, kernel=(3, 3), stride=(2, 2), padding=(1, 1), act="identity",
               is_exit=True)
    return v, block


def randwire_regular_front(v: Value, ch: int):
    block = Block(v.node, None, [], None)
    v = conv2d(block, [[v]], out_channels=ch // 2, kernel=(3, 3), stride=(2, 2), padding=(1, 1),
               act="identity", is_exit=True)
    return v, block


def randwire_tail(v: Value):
    block = Block(v.node, None, [], None)
    v = relu(block, [[v]])
    v = conv2d(block, [[v]], out_channels=1280, kernel=(1, 1), act="identity")
    v = pool2d(block, [[v]], pool_type='global_avg', is_exit=True)
    return v, block


def randwire_stage(r: Value, ch: int, n: int, edges: Sequence[Tuple[int, int]]):
    """Build one stage from a DAG given as edges (u, v) with u < v; node indices are a topological order."""
    block = Block(r.node, None, [], None)
    preds = [[] for _ in range(n)]
    has_succ = [False] * n
    for u, v in edges:
        assert u < v
        preds[v].append(u)
        has_succ[u] = True
    outputs: List[Value] = []
    for u in range(n):
        if preds[u]:
            outputs.append(rwconv2d(block, [[outputs[p] for p in sorted(preds[u])]], out_channels=ch))
        else:
            outputs.append(rwconv2d(block, [[r]], out_channels=ch, stride=(2, 2)))
    sinks = [outputs[u] for u in range(n) if not has_succ[u]]
    return identity(block, [sinks], is_exit=True), block


def _randwire(name, front, front_ch, stages, init_seed, init_scheme):
    """``stages``: (channels, number of nodes, edges) per stage."""
    reset_name()
    pv = placeholder(output_shape=(3, 224, 224))
    v, block = front(pv, front_ch)
    blocks = [block]
    for ch, n, edges in stages:
        v, block = randwire_stage(v, ch, n, edges)
        blocks.append(block)
    v, block = randwire_tail(v)
    blocks.append(block)
    graph = Graph(name, pv.node, blocks)
    graph.init_weights(init_seed, init_scheme)
    return graph


def randwire_small(init_seed=None, init_scheme='uniform', graph_seeds=(3, 4, 5)) -> Graph:
    ch = 78
    stages = [(ch << i, 32, watts_strogatz_edges(32, 4, 0.75, graph_seeds[i])) for i in range(3)]
    return _randwire("randwire_small", randwire_small_front, ch, stages, init_seed, init_scheme)


def randwire_large(init_seed=None, init_scheme='uniform', graph_seeds=(2, 3, 4, 5), graph_files=None) -> Graph:
    """
    The reference's large model: 154 / 308 / 616 / 1232 channels on graphs of 16, 32, 32, 32 nodes (k = 4, p = 0.75), which
    are generated from ``graph_seeds`` or read from the four edge-list files ``graph_files``.
    """
    ch = 154
    if graph_files is not None:
        graphs = [read_graph(fname) for fname in graph_files]
    else:
        graphs = [(n, watts_strogatz_edges(n, 4, 0.75, seed)) for n, seed in zip((16, 32, 32, 32), graph_seeds)]
    if len(graphs) != 4:
        raise ValueError('randwire_large has four stages')
    stages = [(ch << i, n, edges) for i, (n, edges) in enumerate(graphs)]
    return _randwire("randwire_large", randwire_regular_front, ch, stages, init_seed, init_scheme)


def randwire_xlarge(init_seed=None, init_scheme='uniform', graph_seed=0, graph_file=None) -> Graph:
    """One stage of 320 nodes (k = 20, p = 0.75) at 154 channels: the graph the reference counts schedule-search states on."""
    ch = 154
    n, edges = read_graph(graph_file) if graph_file is not None else (320, watts_strogatz_edges(320, 20, 0.75, graph_seed))
    return _randwire("randwire_xlarge", randwire_regular_front, ch, [(ch, n, edges)], init_seed, init_scheme)
