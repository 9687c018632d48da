"""Stand-alone activation / elementwise layers, the kind ``chimera.graph_fusion`` folds into the
chain that produces their input (reference: ``is_act_layer`` / ``is_elem_layer`` in
python/ditto/auto_compute/nn/module, used by python/ditto/chimera/graph_fusion.py:32-35)."""
from .... import te

ACT_KINDS = ("relu", "gelu", "tanh", "sigmoid")
ELEM_KINDS = ("add", "mul")


def _elementwise(kind, tensors, name):
    x = tensors[0]
    for t in tensors[1:]:
        assert tuple(t.shape) == tuple(x.shape) and t.dtype == x.dtype, "elementwise operands must match"
    return te.compute(list(x.shape), name, x.dtype, kind, lambda *ax: [(t, list(ax)) for t in tensors],
                      axis_names=["i%d" % i for i in range(len(x.shape))])


def activation(x, kind="relu", name=None):
    """One activation op over ``x``; ``x`` is usually a fresh placeholder that a graph edge connects to
    the producing layer's output."""
    assert kind in ACT_KINDS, "activation must be one of %s" % (ACT_KINDS,)
    return _elementwise(kind, [x], name or kind)


def ReLU(x, name="relu"):
    return activation(x, "relu", name)


def elementwise(a, b, kind="add", name=None):
    assert kind in ELEM_KINDS, "elementwise op must be one of %s" % (ELEM_KINDS,)
    return _elementwise(kind, [a, b], name or kind)
