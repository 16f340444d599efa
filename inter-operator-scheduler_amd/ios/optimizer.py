"""
Dynamic-programming search for an inter-operator schedule.

For every block (or every part of a large block) the search works on sets of operators encoded as bit
masks.  ``best(S)`` is the cheapest way to execute the operator set ``S`` (which is always closed under
predecessors inside the part): pick an *ending* ``E`` of ``S`` -- a subset closed under successors -- run
it as the last stage and recurse on ``S - E``.  Two kinds of stages exist:

* ``parallel``: ``E`` is a union of at most ``max_num_groups`` pairwise independent groups, each group
  being one operator together with all of its successors inside ``S`` (at most ``max_group_size``
  operators); groups run concurrently on different streams;
* ``merge``: ``E`` is a set of sink convolutions that read the same tensor with the same stride and
  activation; they are replaced by one convolution whose filters are stacked along the output channels.

Stage costs come from a ``CostModel`` and are memoised per operator set.  After the search the chosen
stages are replayed to build a new graph whose blocks carry the schedule.

This is the algorithm of reference python/ios/optimizer.py (optimize :37-194, ending_iterator :450-510,
dop :513-593, check_merge :245-278, construct :609-745), re-implemented around a per-part search object.
Candidates are enumerated in the same order (merge candidates first, then endings with chain 0 as the
fastest digit) and a candidate replaces the incumbent only when strictly cheaper.  The chain
decomposition picks, among equally long chains, the one starting at the lowest operator index, so
schedules under exactly equal costs may differ from the reference's choice.
"""
import itertools
from typing import Dict, List, Optional, Sequence, Set, Tuple

import numpy as np

from ios.cost_model import CostModel, IOSCostModel, RandomCostModel
from ios.ir import Block, Conv, Graph, Node, Placeholder, Sequential, Value
from ios.utils import bits_of, iter_subset, mask_of

IGraph = Dict[int, List[int]]
Stage = Tuple[List[List[int]], str]


# ------------------------------------------------------------------------------------------------
# small graph utilities on index graphs {u: [successors]}
# ------------------------------------------------------------------------------------------------
def build_graph(nodes: Sequence[Node], nid: Dict[Node, int]) -> IGraph:
    """Successor lists restricted to ``nodes``, expressed with the block-wide indices ``nid``."""
    members = set(nodes)
    graph: IGraph = {}
    for node in nodes:
        succ = {nid[use[0]] for use in node.uses if use[0] in members}
        graph[nid[node]] = sorted(succ)
    return graph


def topological_order(graph: IGraph) -> List[int]:
    indeg = {u: 0 for u in graph}
    for u in graph:
        for v in graph[u]:
            indeg[v] += 1
    ready = sorted(u for u in graph if indeg[u] == 0)
    order = []
    while ready:
        u = ready.pop()
        order.append(u)
        for v in graph[u]:
            indeg[v] -= 1
            if indeg[v] == 0:
                ready.append(v)
    assert len(order) == len(graph), 'the operator graph has a cycle'
    return order


def graph_transitive_closure(graph: IGraph, include_self=False) -> Dict[int, Set[int]]:
    closure: Dict[int, Set[int]] = {u: set() for u in graph}
    for u in reversed(topological_order(graph)):
        if include_self:
            closure[u].add(u)
        for v in graph[u]:
            closure[u].add(v)
            closure[u] |= closure[v]
    return closure


def longest_chain(graph: IGraph) -> List[int]:
    depth = {u: 1 for u in graph}
    follow: Dict[int, Optional[int]] = {u: None for u in graph}
    for u in reversed(topological_order(graph)):
        for v in graph[u]:
            if depth[v] + 1 > depth[u]:
                depth[u] = depth[v] + 1
                follow[u] = v
    head = min(graph, key=lambda u: (-depth[u], u))
    chain = []
    while head is not None:
        chain.append(head)
        head = follow[head]
    return chain


def graph_chain_decomposition(graph: IGraph) -> List[List[int]]:
    """Peel longest chains off the transitive closure until no operator is left."""
    closure = graph_transitive_closure(graph)
    reach: IGraph = {u: sorted(closure[u]) for u in graph}
    chains = []
    while reach:
        chain = longest_chain(reach)
        chains.append(chain)
        gone = set(chain)
        reach = {u: [v for v in succ if v not in gone] for u, succ in reach.items() if u not in gone}
    return chains


def count_bits(s: int) -> int:
    return bin(s).count('1')


def state2iset(s: int) -> List[int]:
    return bits_of(s)


def state2nset(s: int, idn: Dict[int, Node]) -> List[Node]:
    return [idn[i] for i in bits_of(s)]


# ------------------------------------------------------------------------------------------------
# merge rule
# ------------------------------------------------------------------------------------------------
def check_merge(s: int, idn: Dict[int, Node]) -> bool:
    """
    A set of operators may be merged when it is a single operator, or when all are ungrouped
    convolutions with one and the same input value, equal input/output resolution, stride and activation.
    """
    nodes = state2nset(s, idn)
    if len(nodes) == 1:
        return True
    if not all(isinstance(node, Conv) for node in nodes):
        return False
    first = nodes[0]
    # (the reference tests groups and inputs from the second operator on, optimizer.py:259-277; a grouped first convolution
    # would be stacked as if it were dense, so it is refused here; further input terms of the first one are merged correctly)
    if first.groups != 1:
        return False
    for node in nodes[1:]:
        if tuple(node.input_shape[1:]) != tuple(first.input_shape[1:]):
            return False
        if tuple(node.output_shape[1:]) != tuple(first.output_shape[1:]):
            return False
        if tuple(node.stride) != tuple(first.stride):
            return False
        if node.groups != 1 or node.act != first.act:
            return False
        if len(node.inputs) != 1 or len(node.inputs[0]) != 1 or not (node.inputs[0][0] == first.inputs[0][0]):
            return False
    return True


def merged_conv_geometry(convs: Sequence[Conv]):
    kernel = (max(c.kernel[0] for c in convs), max(c.kernel[1] for c in convs))
    padding = (max(c.padding[0] for c in convs), max(c.padding[1] for c in convs))
    stride = (convs[0].stride[0], convs[0].stride[1])
    return sum(c.out_channels for c in convs), kernel, stride, padding


def get_input(nodes: Sequence[Node], block: Block, nid, idn) -> List[List[Value]]:
    """Union of the terms of ``nodes`` without duplicates, ordered by (term length, producer indices)."""
    keyed = {}
    for node in nodes:
        for term in node.inputs:
            key = tuple((-1 if v.node is block.enter_node else nid[v.node], v.begin, v.end) for v in term)
            keyed[key] = term
    ordered = sorted(keyed, key=lambda key: (len(key), key))
    return [[Value(block.enter_node if i == -1 else idn[i], b, e) for i, b, e in key] for key in ordered]


# ------------------------------------------------------------------------------------------------
# search over one part of a block
# ------------------------------------------------------------------------------------------------
class _PartSearch:
    def __init__(self, block, part_nodes, nid, idn, opt_type, max_group_size, max_num_groups, cost_model,
                 measure_args, debug, progress):
        self.block, self.nid, self.idn = block, nid, idn
        self.use_merge = 'merge' in opt_type
        self.use_parallel = 'parallel' in opt_type
        self.max_group_size, self.max_num_groups = max_group_size, max_num_groups
        self.cost_model, self.measure_args = cost_model, measure_args
        self.debug, self.progress = debug, progress
        self.graph = build_graph(part_nodes, nid)
        self.chains = graph_chain_decomposition(self.graph)
        self.full_state = mask_of(self.graph.keys())
        self.reach = self._reach_masks()
        self.dp: Dict[int, float] = {}
        self.choice: Dict[int, Stage] = {}
        self.merge_latency: Dict[int, float] = {}
        self.parallel_latency: Dict[int, float] = {}
        self.num_schedules: Dict[int, int] = {0: 1}
        self.num_transitions = 0
        self.width = 0

    # -- stage enumeration --------------------------------------------------------------------------
    def _reach_masks(self) -> Dict[int, int]:
        closure = graph_transitive_closure(self.graph, include_self=True)
        return {u: mask_of(closure[u]) for u in closure}

    def endings(self, state: int):
        """Yield every admissible parallel stage of ``state`` as a list of groups (sorted index lists)."""
        # ``state`` is closed under predecessors, so the successors of u inside it are reach[u] & state
        windows = []
        for chain in self.chains:
            end = 0
            for u in chain:
                if not (state >> u) & 1:
                    break
                end += 1
            begin = max(0, end - self.max_group_size)
            window = []
            for u in chain[begin:end]:
                group = self.reach[u] & state
                if count_bits(group) <= self.max_group_size:
                    window.append((u, group))
            windows.append(window)
        # Enumeration order: mixed radix over the chains with chain 0 as the fastest digit and "unused" as
        # the last value of every digit.  The recursion fixes the slowest digit first and abandons a prefix
        # as soon as it has too many or overlapping groups, which skips whole sub-ranges without changing
        # the order of the survivors.
        limit = self.max_num_groups
        chosen: List[int] = []

        def walk(chain_index: int, used: int):
            if chain_index < 0:
                if chosen:
                    # groups are reported in chain order
                    yield [bits_of(group) for group in reversed(chosen)]
                return
            if len(chosen) < limit:
                for _, group in windows[chain_index]:
                    if used & group:
                        continue
                    chosen.append(group)
                    yield from walk(chain_index - 1, used | group)
                    chosen.pop()
            yield from walk(chain_index - 1, used)

        yield from walk(len(windows) - 1, 0)

    # -- stage cost -------------------------------------------------------------------------------
    def _measure(self, stage_nodes: List[List[Node]]) -> float:
        batch_size, warmup, number, repeat = self.measure_args
        return float(np.mean(self.cost_model.get_stage_latency(stage_nodes, batch_size, warmup, number, repeat)))

    def stage_cost(self, stage: Stage) -> float:
        groups, kind = stage
        key = mask_of(itertools.chain(*groups))
        if kind == 'parallel':
            if key not in self.parallel_latency:
                self.parallel_latency[key] = self._measure([[self.idn[u] for u in g] for g in groups])
            return self.parallel_latency[key]
        if kind == 'merge':
            if key not in self.merge_latency:
                convs = state2nset(key, self.idn)
                if len(convs) == 1:
                    probe = convs[0]
                else:
                    out_channels, kernel, stride, padding = merged_conv_geometry(convs)
                    probe = Conv('c', '', inputs=get_input(convs, self.block, self.nid, self.idn),
                                 out_channels=out_channels, kernel=kernel, stride=stride, padding=padding,
                                 groups=convs[0].groups, act=convs[0].act, output_shape=None)
                    probe.infer_shape()
                self.merge_latency[key] = self._measure([[probe]])
            return self.merge_latency[key]
        raise ValueError(kind)

    # -- recursion ----------------------------------------------------------------------------------
    def solve(self, state: int) -> float:
        if state == 0:
            return 0.0
        if state in self.dp:
            return self.dp[state]
        if self.debug:
            self.num_schedules[state] = 0
        best = 1e19
        if self.use_merge:
            sinks = mask_of(u for u in bits_of(state) if self.reach[u] & state == 1 << u)
            for sub in iter_subset(sinks):
                if check_merge(sub, self.idn):
                    best = self._consider(state, ([[u] for u in bits_of(sub)], 'merge'), sub, best)
        if self.use_parallel:
            for groups in self.endings(state):
                used = mask_of(itertools.chain(*groups))
                best = self._consider(state, (groups, 'parallel'), used, best)
                self.width = max(self.width, len(groups))
        self.dp[state] = best
        if self.progress is not None:
            self.progress.update(1)
        return best

    def _consider(self, state, stage, used, best):
        value = self.solve(state - used) + self.stage_cost(stage)
        if self.debug:
            self.num_transitions += 1
            self.num_schedules[state] += self.num_schedules[state - used]
        if value < best:
            self.choice[state] = stage
            return value
        return best

    def stage_list(self) -> List[Stage]:
        stages = []
        state = self.full_state
        while state:
            stage = self.choice[state]
            stages.append(stage)
            state -= mask_of(itertools.chain(*stage[0]))
        stages.reverse()
        return stages


def get_stage_list(ep: Dict[int, Stage], s: int) -> List[Stage]:
    """Stages from the per-state choices ``ep``, first stage first."""
    out = []
    while s:
        out.append(ep[s])
        s -= mask_of(itertools.chain(*ep[s][0]))
    return out[::-1]


# ------------------------------------------------------------------------------------------------
# rebuilding the graph
# ------------------------------------------------------------------------------------------------
def _fuse_adjacent_slices(terms: List[List[Value]]) -> List[List[Value]]:
    """Join neighbouring single-value terms that are consecutive channel slices of one tensor."""
    fused: List[List[Value]] = []
    for term in terms:
        if fused and len(term) == 1 and len(fused[-1]) == 1:
            prev, cur = fused[-1][0], term[0]
            if prev.node == cur.node and prev.end == cur.begin:
                fused[-1] = [Value(prev.node, prev.begin, cur.end)]
                continue
        fused.append(term)
    return fused


def construct(stage_list: List[Stage], block: Block, constructed_blocks: List[Block], graph_enter, idn, nid,
              compute_weight) -> Block:
    """Replay ``stage_list`` into a new block: operators are cloned, merged stages become one convolution."""
    new_enter = constructed_blocks[-1].exit_node if constructed_blocks else graph_enter
    # old operator -> (new operator, first channel, end channel) holding its result
    located = {block.enter_node: (new_enter, 0, new_enter.output_shape[0])}
    inner_nodes: List[Node] = []
    stages: List[List[List[str]]] = []

    def relocate(terms):
        out = []
        for term in terms:
            new_term = []
            for v in term:
                node, base, _ = located[v.node]
                new_term.append(Value(node, base + v.begin, base + v.end))
            out.append(new_term)
        return _fuse_adjacent_slices(out)

    def clone(old: Node) -> Node:
        config = old.export_config()
        if isinstance(old, Sequential):
            config['nodes'][0]['inputs'] = []
            new = Node.from_config(config, {})
            new.nodes[0].inputs = relocate(old.nodes[0].inputs)
            new.inputs = new.nodes[0].inputs
            pairs = list(zip(new.nodes, old.nodes))
        else:
            config['inputs'] = []
            new = Node.from_config(config, {})
            new.inputs = relocate(old.inputs)
            pairs = [(new, old)]
        new._register_uses()
        if compute_weight:
            for dst, src in pairs:
                if isinstance(dst, Conv):
                    dst.weight, dst.bias = src.weight.copy(), src.bias.copy()
        new.infer_shape()
        located[old] = (new, 0, new.output_shape[0])
        return new

    def merge(convs: List[Conv]) -> Node:
        """
        One convolution for all of ``convs`` (reference optimizer.py:662-711): its input concatenates the distinct input
        terms of the merged convolutions, its filters hold every convolution's filters in the rows of its output channels
        and the columns of its own terms (zeros elsewhere), smaller kernels centred in the common window.  ``check_merge``
        admits convolutions that read one and the same value; like the reference's it does not look at the inputs of the
        first one, which may therefore bring further terms along.
        """
        out_channels, kernel, stride, padding = merged_conv_geometry(convs)
        terms = get_input(convs, block, nid, idn)

        def key_of(term):
            return tuple((id(v.node), v.begin, v.end) for v in term)

        begin_of, at = {}, 0
        for term in terms:
            begin_of[key_of(term)] = at
            at += term[0].length
        new = Conv(convs[0].name, ' '.join(c.hint_name for c in convs), None, out_channels, kernel, stride,
                   padding, 1, convs[0].act, None)
        new.inputs = relocate(terms)      # (joins neighbouring slices; the channel order stays)
        new._register_uses()
        new.infer_shape()
        if compute_weight:
            new.weight = np.zeros(new.weight_shape, dtype=np.float32)
            new.bias = np.zeros(new.bias_shape, dtype=np.float32)
        first = 0
        for conv in convs:
            last = first + conv.out_channels
            if compute_weight:
                # smaller kernels sit centred inside the common kernel window, zeros around them
                r0 = (kernel[0] - conv.kernel[0]) // 2
                c0 = (kernel[1] - conv.kernel[1]) // 2
                own = 0
                for term in conv.inputs:
                    width = term[0].length
                    column = begin_of[key_of(term)]
                    new.weight[first:last, column:column + width, r0:r0 + conv.kernel[0], c0:c0 + conv.kernel[1]] += \
                        conv.weight[:, own:own + width]
                    own += width
                new.bias[first:last] = conv.bias
            located[conv] = (new, first, last)
            first = last
        return new

    for groups, kind in stage_list:
        if kind == 'merge' and len(groups) > 1:
            convs = [idn[i] for i in itertools.chain(*groups)]
            assert all(isinstance(c, Conv) for c in convs)
            new = merge(convs)
            inner_nodes.append(new)
            stages.append([[new.name]])
        else:
            stage_names = []
            for group in groups:
                clones = [clone(idn[i]) for i in group]
                inner_nodes.extend(clones)
                stage_names.append([c.name for c in clones])
            stages.append(stage_names)
    new_exit = inner_nodes.pop()
    return Block(new_enter, new_exit, inner_nodes, stages)


# ------------------------------------------------------------------------------------------------
# public entry points
# ------------------------------------------------------------------------------------------------
def optimize(graph: Graph,
             batch_size=1,
             cost_model: Optional[CostModel] = None,
             opt_type: str = 'dp_parallel_merge',
             warmup=2, number=6, repeat=6,
             max_num_groups=8, max_part_size=100, compute_weight=False, max_group_size=3,
             debug_dp_info=None, verbose=False) -> Graph:
    """
    Search a schedule for ``graph`` and return a new graph carrying it (signature of reference
    optimizer.py:37-43).

    opt_type: 'dp_parallel' (concurrent groups only), 'dp_merge' (operator merge only) or
        'dp_parallel_merge' (both).
    cost_model: prices candidate stages; defaults to measurements on the device.
    warmup/number/repeat: measurement parameters handed to the cost model.
    max_num_groups / max_group_size: pruning limits (groups per stage, operators per group).
    max_part_size: blocks without explicit ``parts`` are cut into consecutive parts of this many operators.
    compute_weight: also produce weights for the new graph (needed for inference with merged convolutions).
    debug_dp_info: optional dict that receives per-part statistics ('#states', '#transitions',
        '#schedules', 'width', '#operators') and the tables 'dp' and 'stage_latency'.
    """
    assert 'parallel' in opt_type or 'merge' in opt_type
    if cost_model is None:
        cost_model = IOSCostModel()
    debug = debug_dp_info is not None
    if debug:
        assert isinstance(debug_dp_info, dict)
        for key in ('dp', 'stage_latency'):
            debug_dp_info[key] = {}
        for key in ('#states', '#transitions', '#schedules', 'width', '#operators', 'meta'):
            debug_dp_info[key] = []
    progress = None
    if verbose:
        print(f'optimize {opt_type} on {graph.name}')
        try:
            from tqdm import tqdm
            progress = tqdm(desc='states')
        except ImportError:
            progress = None

    graph_enter = Placeholder(graph.input.name, graph.input.hint_name, graph.input.output_shape)
    graph_enter.output_shape = graph.enter_node.output_shape
    measure_args = (batch_size, warmup, number, repeat)
    new_blocks: List[Block] = []
    for block in graph.blocks:
        members = block.inner_nodes + [block.exit_node]
        nid = {node: i for i, node in enumerate(members)}
        idn = dict(enumerate(members))
        parts = block.parts
        if parts is None:
            parts = [members[i:i + max_part_size] for i in range(0, len(members), max_part_size)]
        stage_list: List[Stage] = []
        for part in parts:
            search = _PartSearch(block, part, nid, idn, opt_type, max_group_size, max_num_groups, cost_model,
                                 measure_args, debug, progress)
            search.solve(search.full_state)
            stage_list.extend(search.stage_list())
            if debug:
                _record_debug(debug_dp_info, search, part)
        new_blocks.append(construct(stage_list, block, new_blocks, graph_enter, idn, nid, compute_weight))
    if progress is not None:
        progress.close()
    new_graph = Graph(graph.name + "_" + opt_type, graph_enter, new_blocks)
    new_graph.infer_shape()
    return new_graph


def _record_debug(info, search: _PartSearch, part):
    idn = search.idn
    info['#states'].append(len(search.dp))
    info['#transitions'].append(search.num_transitions)
    info['#schedules'].append(search.num_schedules.get(search.full_state, 0))
    info['width'].append(search.width)
    info['#operators'].append(len(part))
    info['meta'].append(dict(search.num_schedules))
    for kind, table in (('parallel', search.parallel_latency), ('merge', search.merge_latency)):
        for key, value in table.items():
            info['stage_latency'][' '.join([kind] + [nd.name for nd in state2nset(key, idn)])] = value
    for state, value in search.dp.items():
        groups, kind = search.choice[state]
        chosen = ' '.join(nd.name for nd in state2nset(mask_of(itertools.chain(*groups)), idn))
        info['dp'][' '.join(nd.name for nd in state2nset(state, idn))] = f'{value:.3f} ({kind} {chosen})'


def graph_dp_summary(graph: Graph, opt_type: str = 'dp_parallel_merge', max_num_groups=8, max_part_size=50,
                     max_group_size=3):
    """Search statistics under a random cost model (reference optimizer.py:17-35); needs no device."""
    info = {}
    optimize(graph, batch_size=1, cost_model=RandomCostModel(), opt_type=opt_type, warmup=1, number=1,
             repeat=1, max_num_groups=max_num_groups, max_part_size=max_part_size,
             max_group_size=max_group_size, compute_weight=False, debug_dp_info=info, verbose=False)
    return info
