"""
Graph drawing (counterpart of reference python/ios/visualizer.py:93).  Drawing needs the optional
``pydot`` package; without it ``draw`` writes the textual schedule next to the requested file name.
"""
import os


def draw(graph, fname, label=None):
    try:
        import pydot  # noqa: F401
    except ImportError:
        pydot = None
    os.makedirs(os.path.dirname(os.path.abspath(fname)) or '.', exist_ok=True)
    if pydot is None:
        with open(os.path.splitext(fname)[0] + '.txt', 'w') as f:
            if label:
                f.write(label + '\n')
            f.write(str(graph) + '\n')
        return
    dot = pydot.Dot(graph_type='digraph', label=label or graph.name)
    for block_index, block in enumerate(graph.blocks):
        cluster = pydot.Cluster(f'block{block_index}', label=f'block {block_index}')
        for node in block.inner_nodes + [block.exit_node]:
            cluster.add_node(pydot.Node(node.name, label=f'{node.hint_name}:{node.type}'))
        dot.add_subgraph(cluster)
    dot.add_node(pydot.Node(graph.input.name, label='input'))
    for node in graph.nodes():
        for term in node.inputs:
            for value in term:
                dot.add_edge(pydot.Edge(value.node.name, node.name))
    dot.write(fname, format=os.path.splitext(fname)[1][1:] or 'png')
