"""Graph-level fusion pass (reference: python/ditto/chimera/graph_fusion.py:4-52).

The reference walks the layers in order and fuses a following activation / elementwise layer into
the layer that produces its input, leaving attention layers alone (they are already one fused
chain).  Here the producer is a fused chain whose kernel has a ReLU slot after the second
contraction (``relu_out`` of both C-ABI descriptors), so fusing a ReLU layer means re-describing
the chain's output op as ``relu_cast`` and dropping the activation layer from the graph.  What
has no slot in a kernel -- other activations, a residual add, an activation behind an attention
layer or behind an output that something else also reads -- is left in the graph as it is.
"""
from .. import te
from ..auto_compute.graph import Layer
from ..auto_compute.nn.functional.elementwise import ACT_KINDS, ELEM_KINDS
from ..auto_compute.nn.module import is_self_attention_layer


def _compute_ops(layer):
    return [op for op in layer.all_ops if isinstance(op, te.ComputeOp)]


def is_act_layer(layer):
    """A layer that is a lone activation op."""
    ops = _compute_ops(layer)
    return len(ops) == 1 and ops[0].kind in ACT_KINDS


def is_elem_layer(layer):
    """A layer that is a lone two-operand elementwise op (e.g. a residual add)."""
    ops = _compute_ops(layer)
    return len(ops) == 1 and ops[0].kind in ELEM_KINDS


def can_fuse_activation(producer, act_layer):
    """ReLU behind a chain whose output op is the plain final cast: the kernels' ``relu_out`` slot."""
    if is_self_attention_layer(producer) or len(producer.ops) != 1 or not is_act_layer(act_layer):
        return False
    if _compute_ops(act_layer)[0].kind != "relu":
        return False
    out = producer.ops[0]
    if not isinstance(out, te.ComputeOp) or out.kind != "unpack_cast" or out.output(0).dtype == "int32":
        return False
    src, dst = out.output(0), act_layer.inputs[0]
    return tuple(src.shape) == tuple(dst.shape) and src.dtype == dst.dtype


def fuse_activation(producer, act_layer):
    """The producer chain with its output op re-described as cast + ReLU (a new layer; the
    producer's contraction ops are shared, not copied)."""
    if not can_fuse_activation(producer, act_layer):
        raise ValueError("layer %s cannot take the activation of %s" % (producer.name, act_layer.name))
    old = producer.ops[0]
    (src, _), = old.accesses
    out = te.compute(list(old.output(0).shape), old.name, old.output(0).dtype, "relu_cast",
                     lambda *ax: [(src, list(ax))], axis_names=[iv.name for iv in old.axis],
                     attrs=dict(old.attrs, fused_activation="relu"))
    return Layer(producer.name + "_relu", [out.op], producer.inputs, producer.weights, producer.const_scalars,
                 producer.const_tensors)


def graph_fusion(graph):
    """Fuse every ReLU layer that is the only reader of a chain layer's output into that chain.
    Returns a new graph (the given one is not modified); a graph with nothing to fuse is returned
    as it is."""
    layers = list(graph.get_all_layers())
    assert len(layers) > 0
    edges = dict(graph.edges)
    outputs = list(graph.graph_outputs)
    fused_any = False
    j = 0
    while j < len(layers):
        act = layers[j]
        src = edges.get((j, 0)) if is_act_layer(act) and len(act.inputs) == 1 else None
        if src is None:
            j += 1
            continue
        i, oi = src
        readers = [c for c, p in edges.items() if p == (i, oi)]
        if oi != 0 or len(readers) != 1 or (i, oi) in outputs or not can_fuse_activation(layers[i], act):
            j += 1
            continue
        layers[i] = fuse_activation(layers[i], act)
        del layers[j]
        # what read the activation now reads the fused chain; indices past the dropped layer shift down
        def remap(li, k):
            if li == j:
                return (i, 0)
            return (li - 1 if li > j else li, k)
        edges = {(c - 1 if c > j else c, k): remap(*p) for (c, k), p in edges.items() if c != j}
        outputs = [remap(*o) for o in outputs]
        fused_any = True
    if not fused_any:
        return graph
    return type(graph)(layers, edges, outputs)
