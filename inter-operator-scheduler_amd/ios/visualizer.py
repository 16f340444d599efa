"""
Graph drawing (counterpart of reference python/ios/visualizer.py:93 ``draw``), without the pydot dependency: the graph is
written as Graphviz DOT text, one cluster per block, one fill colour per stage, an edge per input value (labelled with its
channel range when it is a slice; values that are summed meet in one arrow head).  ``fname`` with the extension ``.dot`` or
``.gv`` receives the text; any other extension is rendered with the ``dot`` program when it is installed, and falls back to
``<fname>.dot`` beside it when it is not.
"""
import os
import shutil
import subprocess

_STAGE_COLOURS = ['lightblue', 'lightgoldenrod1', 'palegreen', 'lightpink', 'lightsalmon', 'plum1', 'khaki', 'paleturquoise',
                  'thistle', 'wheat', 'darkseagreen1', 'lightcyan', 'mistyrose', 'lavender']


def _quote(text) -> str:
    return '"' + str(text).replace('\\', '\\\\').replace('"', '\\"').replace('\n', '\\n') + '"'


def _label(node, stage) -> str:
    lines = [node.type if node.type != 'conv' else f'conv {node.kernel[0]}x{node.kernel[1]}' + (f' g{node.groups}' if node.groups > 1 else '')]
    if node.type == 'pool':
        lines[0] = f'pool {node.pool_type}'
    where = '' if stage is None else f' @ stage {stage}'
    lines.append(f'{node.hint_name}{where}')
    mflops = node.flops() / 1e6 if node.type != 'placeholder' else 0.0
    lines.append(f'{tuple(node.output_shape)}' + (f'  {mflops:.1f} MFLOP' if mflops else ''))
    return '\n'.join(lines)


def to_dot(graph, label=None) -> str:
    """DOT source of ``graph`` with its current schedule (operators without a schedule are drawn uncoloured)."""
    out = ['digraph ' + _quote(graph.name) + ' {', '  rankdir=TB; node [shape=box, style="rounded,filled", fillcolor=white, fontsize=10];',
           '  labelloc=t; label=' + _quote(label or graph.name) + ';',
           '  ' + _quote(graph.input.name) + ' [label=' + _quote(_label(graph.input, None)) + ', shape=oval];']
    stage_number = 0
    for index, block in enumerate(graph.blocks):
        stage_of = {}
        for stage in block.stages or []:
            for group in stage:
                for name in group:
                    stage_of[name] = stage_number
            stage_number += 1
        out.append(f'  subgraph cluster_{index} {{ label="block {index}"; color=gray60;')
        for node in block.inner_nodes + [block.exit_node]:
            stage = stage_of.get(node.name)
            colour = 'white' if stage is None else _STAGE_COLOURS[stage % len(_STAGE_COLOURS)]
            out.append(f'    {_quote(node.name)} [label={_quote(_label(node, stage))}, fillcolor={colour}];')
        out.append('  }')
    for node in graph.nodes():
        if node is graph.input:
            continue
        for term_index, term in enumerate(node.inputs):
            for value in term:
                whole = value.begin == 0 and value.end == value.node.output_shape[0]
                attributes = [] if whole else ['label=' + _quote(f'[{value.begin}:{value.end}]')]
                if len(term) > 1:
                    attributes.append('arrowhead=odot')      # summed with the other values of its term
                if len(node.inputs) > 1:
                    attributes.append('taillabel=' + _quote(term_index))
                out.append(f'  {_quote(value.node.name)} -> {_quote(node.name)}' + (' [' + ', '.join(attributes) + ']' if attributes else '') + ';')
    out.append('}')
    return '\n'.join(out) + '\n'


def draw(graph, fname, label=None):
    """Write a picture of ``graph`` and its schedule to ``fname`` (see the module docstring for the formats)."""
    os.makedirs(os.path.dirname(os.path.abspath(fname)) or '.', exist_ok=True)
    source = to_dot(graph, label)
    extension = os.path.splitext(fname)[1][1:].lower()
    renderer = shutil.which('dot')
    if extension in ('dot', 'gv', ''):
        target = fname if extension else fname + '.dot'
    elif renderer is not None:
        subprocess.run([renderer, '-T' + extension, '-o', fname], input=source.encode(), check=True)
        return fname
    else:
        target = fname + '.dot'
    with open(target, 'w') as f:
        f.write(source)
    return target
