"""Graph-level fusion pass (reference: python/ditto/chimera/graph_fusion.py:4-52).

The reference walks the layers in order and fuses an activation / elementwise layer into its
producer, leaving attention layers alone (they are already one fused chain).  The graphs this
package runs hold fused-chain layers only -- activation and elementwise epilogues are part of the
chain kernels (ReLU on the inter path and after the second contraction) -- so there is nothing to
merge and the pass returns the graph unchanged after checking that it holds no layer it would
have to fuse.
"""
from ..auto_compute.nn.module import is_self_attention_layer

ACT_KINDS = ("relu", "gelu", "tanh", "sigmoid")


def is_act_layer(layer):
    """A layer that is a lone activation op."""
    ops = [op for op in layer.all_ops if getattr(op, "kind", None) is not None]
    return len(ops) == 1 and ops[0].kind in ACT_KINDS


def graph_fusion(graph):
    layers = graph.get_all_layers()
    assert len(layers) > 0
    for layer in layers:
        if not is_self_attention_layer(layer) and is_act_layer(layer):
            raise NotImplementedError(
                "graph_fusion: stand-alone activation layer %s; activations belong on the chain's inter path "
                "or epilogue here" % layer.name)
    return graph
