"""
Computation-graph IR of the inter-operator scheduler.

A network is a ``Graph`` = an input ``Placeholder`` followed by a chain of ``Block`` objects.  A block is
a DAG of operators with one enter operator (owned by the previous block) and one exit operator.  Every
operator reads ``inputs`` = a list of *terms*; a term is a list of ``Value`` channel slices that are
summed, and the terms are concatenated on the channel axis.  A block may carry an execution schedule
``stages``: a list of stages, each a list of groups, each a list of operator names.  Stages run one
after another, groups of one stage run concurrently, operators of one group run in order.

The class names, attributes, method names and the exported JSON documents follow the reference IR
(reference python/ios/ir.py:19-81 Value, :84-242 Node, :245-797 operator classes, :800-977 Block,
:980-1132 Graph) so that graphs and schedules are interchangeable with it.  The implementation is
table driven: every operator class lists its configuration keys once and the base class derives
``export_config`` / ``from_config`` from that list.
"""
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np


class Value:
    """Channel slice ``[begin, end)`` of the output of ``node`` (reference ir.py:19-81)."""
    __slots__ = ['node', 'begin', 'end']

    def __init__(self, node, begin, end):
        self.node = node
        self.begin = begin
        self.end = end

    @property
    def length(self):
        return self.end - self.begin

    @staticmethod
    def from_config(config, name2nodes):
        name, begin, end = config
        return Value(name2nodes[name], begin, end)

    def export_config(self):
        return [self.node.name, self.begin, self.end]

    def __eq__(self, other):
        return (isinstance(other, Value) and self.node == other.node
                and self.begin == other.begin and self.end == other.end)

    def __hash__(self):
        return hash((id(self.node), self.begin, self.end))

    def __repr__(self):
        return f'({self.node.hint_name}:{self.begin}:{self.end})'

    __str__ = __repr__


def _terms_from_config(terms_config, name2node):
    if terms_config is None:
        return None
    return [[Value.from_config(vc, name2node) for vc in term] for term in terms_config]


def _terms_to_config(terms):
    if terms is None:
        return None
    return [[v.export_config() for v in term] for term in terms]


def _window_out(size, kernel, pad, stride):
    # floor formula shared by convolution and pooling (reference ir.py:388-393,538-542)
    if size + 2 * pad < kernel:
        raise ValueError(f'window of {kernel} does not fit an input of {size} with padding {pad}')
    return 1 + (size - kernel + 2 * pad) // stride


class Node:
    """
    Base class of all operators (reference ir.py:84-242).

    ``CONFIG_KEYS`` lists the operator specific attributes that are serialised between ``inputs`` and
    ``output_shape`` in the exported document; ``TYPE`` is the value of the ``type`` key.
    """
    __slots__ = ['type', 'name', 'hint_name', 'inputs', 'output_shape', 'uses']
    TYPE = None
    CONFIG_KEYS: Tuple[str, ...] = ()
    _registry: Dict[str, type] = {}

    def __init__(self, type, name, hint_name, inputs, output_shape):
        self.type = type
        self.name = name
        self.hint_name = hint_name
        self.inputs = inputs
        self.output_shape = output_shape
        self.uses: List[Tuple['Node', int, int]] = []

    def __init_subclass__(cls, **kwargs):
        super().__init_subclass__(**kwargs)
        if cls.TYPE is not None:
            Node._registry[cls.TYPE] = cls

    # ---- (de)serialisation -------------------------------------------------------------------
    @staticmethod
    def from_config(config, name2node):
        """Build the operator described by ``config``; unknown ``type`` raises ValueError."""
        cls = Node._registry.get(config['type'])
        if cls is None:
            raise ValueError(f"unrecognized node type {config['type']}")
        return cls._build(config, name2node)

    @classmethod
    def _build(cls, config, name2node):
        kwargs = {key: config[key] for key in cls.CONFIG_KEYS}
        node = cls(name=config['name'], hint_name=config['hint_name'],
                   inputs=_terms_from_config(config['inputs'], name2node),
                   output_shape=config['output_shape'], **kwargs)
        node._register_uses(name2node)
        return node

    def _register_uses(self, name2node=None):
        for ti, term in enumerate(self.inputs or []):
            for vi, value in enumerate(term):
                producer = value.node if name2node is None else name2node[value.node.name]
                producer.uses.append((self, ti, vi))

    def export_config(self):
        config = {'type': self.type, 'name': self.name, 'hint_name': self.hint_name,
                  'inputs': _terms_to_config(self.inputs)}
        for key in self.CONFIG_KEYS:
            config[key] = getattr(self, key)
        config['output_shape'] = self.output_shape
        return config

    # ---- shapes -------------------------------------------------------------------------------
    @property
    def input_shape(self):
        first = self.inputs[0][0].node.output_shape
        return (sum(term[0].length for term in self.inputs), first[1], first[2])

    def infer_shape(self):
        self.output_shape = self.input_shape

    # ---- analytic costs of the input algebra (reference ir.py:180-215) ---------------------------
    def _term_sizes(self):
        sizes = []
        for term in self.inputs:
            shape = term[0].node.output_shape
            sizes.append(shape[1] * shape[2] * term[0].length)
        return sizes

    def input_flops(self):
        return sum(len(term) * size for term, size in zip(self.inputs, self._term_sizes()))

    def input_memory_access(self):
        sizes = self._term_sizes()
        total = sum(size * len(term) for term, size in zip(self.inputs, sizes) if len(term) > 1)
        if len(self.inputs) > 1:
            total += sum(sizes)
        return total

    def input_kernels(self):
        return sum(1 for term in self.inputs if len(term) > 1) + (1 if len(self.inputs) > 1 else 0)

    def flops(self):
        raise NotImplementedError

    def memory_access(self):
        raise NotImplementedError

    def kernels(self):
        raise NotImplementedError

    # ---- pretty printing ----------------------------------------------------------------------
    def input_readable_str(self, merge_op='+'):
        parts = [merge_op.join(v.node.hint_name for v in term) for term in self.inputs]
        if len(parts) > 1:
            return 'Concat(' + ','.join(parts) + ')'
        return '(' + parts[0] + ')' if len(self.inputs[0]) > 1 else parts[0]

    def readable_lines(self, indent) -> List[str]:
        raise NotImplementedError

    def __repr__(self):
        return self.name


class Placeholder(Node):
    """Graph input (reference ir.py:245-277)."""
    TYPE = 'placeholder'

    def __init__(self, name, hint_name, output_shape):
        super().__init__('placeholder', name, hint_name, [[]], output_shape)

    @classmethod
    def _build(cls, config, name2node):
        return cls(config['name'], config['hint_name'], output_shape=config['output_shape'])

    def export_config(self):
        return {'type': 'placeholder', 'name': self.name, 'hint_name': self.hint_name,
                'output_shape': self.output_shape}

    def infer_shape(self):
        pass

    def flops(self):
        return 0.0

    def memory_access(self):
        return 0.0

    def kernels(self):
        return 0

    def readable_lines(self, indent):
        return [f'[{self.hint_name}]Placeholder']


class Conv(Node):
    """
    2-D cross-correlation with bias and fused activation (reference ir.py:280-396).

    ``weight`` has shape (out_channels, in_channels // groups, kh, kw), ``bias`` (out_channels,); both
    may stay ``None`` for latency measurements and must be set before inference.
    """
    __slots__ = ['out_channels', 'kernel', 'stride', 'padding', 'groups', 'act', 'weight', 'bias']
    TYPE = 'conv'
    CONFIG_KEYS = ('out_channels', 'kernel', 'stride', 'padding', 'groups', 'act')
    ACTS = ('relu', 'sigmoid', 'tanh', 'identity')

    def __init__(self, name, hint_name, inputs, out_channels, kernel, stride, padding, groups, act,
                 output_shape):
        super().__init__('conv', name, hint_name, inputs, output_shape)
        assert act in Conv.ACTS
        self.out_channels = out_channels
        self.kernel = kernel
        self.stride = stride
        self.padding = padding
        self.groups = groups
        self.act = act
        self.weight: Optional[np.ndarray] = None
        self.bias: Optional[np.ndarray] = None

    @property
    def weight_shape(self):
        return (self.out_channels, self.input_shape[0] // self.groups, self.kernel[0], self.kernel[1])

    @property
    def bias_shape(self):
        return self.out_channels,

    @property
    def fan_in(self):
        return self.kernel[0] * self.kernel[1] * self.input_shape[0] // self.groups

    def init_weights(self, rng=None, scheme='uniform', gain=1.0):
        """
        Fill ``weight``/``bias``.

        scheme 'uniform' draws both from U(-1/sqrt(fan_in), 1/sqrt(fan_in)) like the reference
        (ir.py:360-363); 'he_normal' draws weight ~ N(0, 2/fan_in) and sets bias to zero; 'he_normal_bias' adds a
        bias ~ N(0, 0.1^2); 'bn_folded' is a convolution with a batch normalisation folded into it
        (w' = w * gamma / sigma, b' = beta - mu * gamma / sigma): weight ~ N(0, gain/fan_in) times a per-channel
        factor from U(0.75, 1.25), bias ~ N(0, 0.1^2), where the caller passes the ``gain`` that stands for
        1 / sigma^2 of the convolution's unit-variance inputs (see Graph.init_weights).
        ``rng`` is a ``numpy.random.Generator``; ``None`` uses the global numpy state.
        """
        normal = np.random.standard_normal if rng is None else rng.standard_normal
        uniform = np.random.uniform if rng is None else rng.uniform
        if scheme == 'uniform':
            bound = 1.0 / np.sqrt(self.fan_in)
            self.weight = uniform(low=-bound, high=bound, size=self.weight_shape).astype(np.float32)
            self.bias = uniform(low=-bound, high=bound, size=self.bias_shape).astype(np.float32)
        elif scheme in ('he_normal', 'he_normal_bias'):
            std = np.sqrt(2.0 / self.fan_in)
            self.weight = (normal(size=self.weight_shape) * std).astype(np.float32)
            if scheme == 'he_normal':
                self.bias = np.zeros(self.bias_shape, dtype=np.float32)
            else:
                self.bias = (normal(size=self.bias_shape) * 0.1).astype(np.float32)
        elif scheme == 'bn_folded':
            std = np.sqrt(gain / self.fan_in)
            per_channel = uniform(low=0.75, high=1.25, size=(self.out_channels, 1, 1, 1))
            self.weight = (normal(size=self.weight_shape) * std * per_channel).astype(np.float32)
            self.bias = (normal(size=self.bias_shape) * 0.1).astype(np.float32)
        else:
            raise ValueError(f'unknown init scheme {scheme}')

    def infer_shape(self):
        _, h, w = self.input_shape
        self.output_shape = (self.out_channels,
                             _window_out(h, self.kernel[0], self.padding[0], self.stride[0]),
                             _window_out(w, self.kernel[1], self.padding[1], self.stride[1]))

    def flops(self):
        # the reference counts one multiply-accumulate as one operation plus one for the bias
        per_output = 1 + self.fan_in
        return int(np.prod(self.output_shape)) * per_output + self.input_flops()

    def memory_access(self):
        return int(np.prod(self.input_shape)) + self.input_memory_access()

    def kernels(self):
        return 1 + self.input_kernels()

    def readable_lines(self, indent):
        return [f'[{self.hint_name}]Conv2d({self.input_readable_str()})']


class Sequential(Node):
    """Compound operator: ``nodes`` run in order, child i+1 reads child i (reference ir.py:399-461)."""
    __slots__ = ['nodes']
    TYPE = 'sequential'

    def __init__(self, name, hint_name, nodes: List[Node], output_shape):
        super().__init__('sequential', name, hint_name, nodes[0].inputs, output_shape)
        self.nodes = nodes

    @classmethod
    def _build(cls, config, name2node):
        children = []
        for child_config in config['nodes']:
            child = Node.from_config(child_config, name2node)
            name2node[child.name] = child
            children.append(child)
        node = cls(config['name'], config['hint_name'], children, config['output_shape'])
        node._register_uses(name2node)
        return node

    def export_config(self):
        return {'type': self.type, 'name': self.name, 'hint_name': self.hint_name,
                'nodes': [child.export_config() for child in self.nodes],
                'output_shape': self.output_shape}

    def infer_shape(self):
        for child in self.nodes:
            child.infer_shape()
        self.output_shape = self.nodes[-1].output_shape

    def flops(self):
        return sum(child.flops() for child in self.nodes)

    def memory_access(self):
        return sum(child.memory_access() for child in self.nodes)

    def kernels(self):
        return sum(child.kernels() for child in self.nodes)

    def readable_lines(self, indent):
        lines = [f'[{self.hint_name}]Sequential(']
        for child in self.nodes:
            lines.extend(' ' * indent + line for line in child.readable_lines(indent))
        lines.append(')')
        return lines


class Pool(Node):
    """
    Pooling, ``pool_type`` in max / avg / global_max / global_avg (reference ir.py:464-564).  The
    average divides by kh*kw everywhere (padding counts as zeros).
    """
    __slots__ = ['pool_type', 'kernel', 'stride', 'padding']
    TYPE = 'pool'
    CONFIG_KEYS = ('pool_type', 'kernel', 'stride', 'padding')
    _PRETTY = {'max': 'MaxPool2d', 'avg': 'AvgPool2d',
               'global_max': 'GlobalMaxPool2d', 'global_avg': 'GlobalAvgPool2d'}

    def __init__(self, name, hint_name, inputs, pool_type, kernel, stride, padding, output_shape):
        super().__init__('pool', name, hint_name, inputs, output_shape)
        self.pool_type = pool_type
        self.kernel = kernel
        self.stride = stride
        self.padding = padding

    def infer_shape(self):
        c, h, w = self.input_shape
        if 'global' in self.pool_type:
            # the runtime treats every global_* pool as a window over the whole map
            self.stride = (1, 1)
            self.padding = (0, 0)
            self.kernel = (h, w)
        self.output_shape = [c,
                             _window_out(h, self.kernel[0], self.padding[0], self.stride[0]),
                             _window_out(w, self.kernel[1], self.padding[1], self.stride[1])]

    def flops(self):
        size = int(np.prod(self.input_shape))
        if 'global' in self.pool_type:
            return size + self.input_flops()
        return size * self.kernel[0] * self.kernel[1] + self.input_flops()

    def memory_access(self):
        return int(np.prod(self.input_shape)) + self.input_memory_access()

    def kernels(self):
        return 1 + self.input_kernels()

    def readable_lines(self, indent):
        return [f'[{self.hint_name}]{Pool._PRETTY[self.pool_type]}({self.input_readable_str()})']


class Element(Node):
    """Element-wise add / mul of the values of its single term (reference ir.py:567-629)."""
    __slots__ = ['op_type']
    TYPE = 'element'
    CONFIG_KEYS = ('op_type',)

    def __init__(self, name, hint_name, inputs, op_type, output_shape):
        super().__init__('element', name, hint_name, inputs, output_shape)
        self.op_type = op_type

    def flops(self):
        return 0.0 + self.input_flops()

    def memory_access(self):
        return 0.0 + self.input_memory_access()

    def kernels(self):
        return self.input_kernels()

    def readable_lines(self, indent):
        return [f"[{self.hint_name}]{self.input_readable_str('*' if self.op_type == 'mul' else '+')}"]


class Identity(Node):
    """Identity of its input algebra, i.e. the add / concat operator (reference ir.py:632-682)."""
    TYPE = 'identity'

    def __init__(self, name, hint_name, inputs, output_shape):
        super().__init__('identity', name, hint_name, inputs, output_shape)

    def flops(self):
        return 0.0 + self.input_flops()

    def memory_access(self):
        return 0.0 + self.input_memory_access()

    def kernels(self):
        return self.input_kernels()

    def readable_lines(self, indent):
        text = self.input_readable_str()
        if not text.startswith('C'):
            text = '(' + text + ')'
        return [f'[{self.hint_name}]{text}']


class _Pointwise(Node):
    def flops(self):
        return 4 * int(np.prod(self.input_shape)) + self.input_flops()

    def memory_access(self):
        return int(np.prod(self.input_shape)) + self.input_memory_access()

    def kernels(self):
        return 1 + self.input_kernels()


class Activation(_Pointwise):
    """relu / tanh / sigmoid, optionally in place (reference ir.py:685-747)."""
    __slots__ = ['act_type', 'inplace']
    TYPE = 'activation'
    CONFIG_KEYS = ('act_type', 'inplace')

    def __init__(self, name, hint_name, inputs, act_type, inplace, output_shape):
        super().__init__('activation', name, hint_name, inputs, output_shape)
        self.act_type = act_type
        self.inplace = inplace

    def readable_lines(self, indent):
        return [f'{self.act_type.capitalize()}@{self.hint_name}({self.input_readable_str()})']


class Relu(_Pointwise):
    """ReLU (reference ir.py:750-797)."""
    TYPE = 'relu'

    def __init__(self, name, hint_name, inputs, output_shape):
        super().__init__('relu', name, hint_name, inputs, output_shape)

    def readable_lines(self, indent):
        return [f'[{self.hint_name}]Relu({self.input_readable_str()})']


class Block:
    """A DAG of operators plus its schedule (reference ir.py:800-977)."""
    __slots__ = ['enter_node', 'exit_node', 'inner_nodes', 'stages', 'parts']

    def __init__(self, enter_node, exit_node=None, inner_nodes=None, stages=None):
        self.enter_node: Optional[Node] = enter_node
        self.exit_node: Optional[Node] = exit_node
        self.inner_nodes: List[Node] = [] if inner_nodes is None else inner_nodes
        self.stages = stages
        self.parts = None

    @property
    def all_nodes(self) -> List[Node]:
        return self.inner_nodes + [self.exit_node]

    @staticmethod
    def from_config(config, name2node):
        enter_node = name2node[config['enter_name']]
        inner_nodes = []
        for inner_config in config['inner_nodes']:
            node = Node.from_config(inner_config, name2node)
            name2node[node.name] = node
            inner_nodes.append(node)
        exit_node = Node.from_config(config['exit_node'], name2node)
        name2node[exit_node.name] = exit_node
        return Block(enter_node, exit_node, inner_nodes, config['stages'])

    def export_config(self):
        return {'enter_name': self.enter_node.name,
                'enter_node': self.enter_node.export_config(),
                'inner_nodes': [node.export_config() for node in self.inner_nodes],
                'exit_node': self.exit_node.export_config(),
                'stages': self.stages}

    def sequential_schedule(self):
        """One operator per stage in definition order."""
        self.stages = [[[node.name]] for node in self.all_nodes]

    def greedy_schedule(self, max_num_stream):
        """
        Level-by-level schedule: every stage takes up to ``max_num_stream`` operators whose inputs are
        all computed; operators that do not fit wait for the next stage (reference ir.py:876-907).
        """
        members = self.all_nodes
        member_set = set(members)
        pending = {node: sum(len(term) for term in node.inputs) for node in members}
        ready: List[Node] = [node for node in members if len(node.inputs) == 0]
        frontier: List[Node] = [self.enter_node] + ready
        self.stages = []
        while frontier:
            runnable = [node for node in frontier if node is not self.enter_node]
            held_back: List[Node] = []
            if runnable:
                held_back = runnable[max_num_stream:]
                self.stages.append([[node.name] for node in runnable[:max_num_stream]])
            finished = [node for node in frontier if node not in held_back]
            released = []
            for node in finished:
                if node is self.exit_node:
                    continue
                for consumer, _, _ in node.uses:
                    if consumer not in member_set:
                        continue
                    pending[consumer] -= 1
                    if pending[consumer] == 0:
                        released.append(consumer)
            frontier = held_back + released
        assert sum(len(stage) for stage in self.stages) == len(members)

    def flops(self):
        return sum(node.flops() for node in self.all_nodes)

    def memory_access(self):
        return sum(node.memory_access() for node in self.all_nodes)

    def kernels(self):
        return sum(node.kernels() for node in self.all_nodes)

    def schedule_operators(self):
        return len(self.all_nodes)

    def readable_lines(self, indent=0):
        by_name: Dict[str, Node] = {node.name: node for node in self.all_nodes}
        pad = ' ' * indent

        def wrapped(title, bodies):
            lines = [title]
            for body in bodies:
                lines.extend(pad + line for line in body)
            lines.append(')')
            return lines

        def group_lines(group):
            bodies = [by_name[name].readable_lines(indent) for name in group]
            return bodies[0] if len(group) == 1 else wrapped('Sequential (', bodies)

        lines = []
        for stage in self.stages:
            bodies = [group_lines(group) for group in stage]
            lines.extend(bodies[0] if len(stage) == 1 else wrapped('Parallel(', bodies))
        return lines


class Graph:
    """A chain of blocks with a single input placeholder (reference ir.py:980-1132)."""
    __slots__ = ['name', 'input', 'input_shape', 'blocks']

    def __init__(self, name, input, blocks):
        self.name = name
        self.input: Placeholder = input
        self.blocks: List[Block] = blocks

    def nodes(self) -> Iterable[Node]:
        """All schedule units in topological (definition) order, starting with the graph input."""
        if not self.blocks:
            return
        yield self.blocks[0].enter_node
        for block in self.blocks:
            yield from block.inner_nodes
            yield block.exit_node

    @property
    def enter_node(self) -> Node:
        return self.blocks[0].enter_node

    @property
    def exit_node(self) -> Node:
        return self.blocks[-1].exit_node

    @staticmethod
    def from_config(config):
        name2node: Dict[str, Node] = {}
        input = Placeholder._build(config['input'], name2node)
        name2node[input.name] = input
        blocks = [Block.from_config(block_config, name2node) for block_config in config['blocks']]
        graph = Graph(config['name'], input, blocks)
        graph.infer_shape()
        return graph

    def export_config(self):
        return {'name': self.name, 'input': self.input.export_config(),
                'blocks': [block.export_config() for block in self.blocks]}

    def infer_shape(self):
        enter = self.blocks[0].enter_node
        for node in self.nodes():
            if node is not enter:
                node.infer_shape()

    def conv_nodes(self) -> List[Conv]:
        """Every convolution, including those nested in Sequential operators, in graph order."""
        found: List[Conv] = []

        def visit(nodes):
            for node in nodes:
                if isinstance(node, Conv):
                    found.append(node)
                elif isinstance(node, Sequential):
                    visit(node.nodes)

        visit(self.nodes())
        return found

    def init_weights(self, seed=None, scheme='uniform'):
        """
        Initialise every convolution.  Without arguments this is the reference behaviour
        (ir.py:1057-1070: unseeded uniform weights and biases).  With ``seed`` the draws come from
        ``numpy.random.default_rng(seed)`` in graph order; ``scheme='he_normal'`` gives N(0, 2/fan_in)
        weights and zero bias, ``'he_normal_bias'`` the same with a small seeded bias.

        ``scheme='bn_folded'`` stands for networks whose convolutions carry a folded batch normalisation
        (RandWire): every convolution is scaled so that unit-variance inputs give unit-variance outputs, i.e. its
        weight variance is gain / fan_in with gain = 1 / (second moment of its input: sums add, a ReLU halves),
        which is what dividing by the batch statistics' sigma would do.  Activations then stay O(1) at any depth
        and fan-in.
        """
        rng = None if seed is None else np.random.default_rng(seed)
        if scheme != 'bn_folded':
            for conv in self.conv_nodes():
                conv.init_weights(rng, scheme)
            return

        # second moment of every operator's output under this initialisation, for unit-variance network input:
        # a convolution normalises to 1, a sum adds, a ReLU of a zero-mean value halves, concatenation takes the
        # largest term, pooling keeps it
        moment: Dict[str, float] = {}

        def of_terms(terms) -> float:
            return max(sum(moment_of(v.node) for v in term) for term in terms)

        def moment_of(node: Node) -> float:
            if node.name not in moment:
                if isinstance(node, (Placeholder, Conv)):
                    value = 1.0
                elif isinstance(node, Sequential):
                    value = moment_of(node.nodes[-1])
                elif isinstance(node, Relu) or (isinstance(node, Activation) and node.act_type == 'relu'):
                    value = of_terms(node.inputs) / 2.0
                elif isinstance(node, Activation):
                    value = 1.0      # tanh and sigmoid are bounded
                else:                # identity (sums and concatenations), element, pool
                    value = of_terms(node.inputs)
                moment[node.name] = value
            return moment[node.name]

        for conv in self.conv_nodes():
            conv.init_weights(rng, scheme, gain=1.0 / of_terms(conv.inputs))

    def sequential_schedule(self):
        for block in self.blocks:
            block.sequential_schedule()

    def greedy_schedule(self, max_num_stream=10):
        for block in self.blocks:
            block.greedy_schedule(max_num_stream)

    def flops(self):
        return sum(block.flops() for block in self.blocks)

    def memory_access(self):
        return sum(block.memory_access() for block in self.blocks)

    def kernels(self):
        return sum(block.kernels() for block in self.blocks)

    def schedule_operators(self):
        return sum(block.schedule_operators() for block in self.blocks)

    def readable_lines(self, indent=0):
        lines = ['Sequential(']
        for block in self.blocks:
            lines.extend(' ' * indent + line for line in block.readable_lines(indent))
        lines.append(')')
        return lines

    def __str__(self):
        return '\n'.join(self.readable_lines(2))
