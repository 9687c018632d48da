"""``layer`` / ``Layer``: wraps a chain DAG and fixes the argument order of the built
function (reference: python/ditto/auto_compute/graph.py:48-203, src/auto_compute/graph.cc:406).
"""
from .. import te


class Layer:
    """A layer = output ops + the tensors that feed them.

    ``schedule_tensors`` is the positional order ``inputs, weights, const_scalars,
    const_tensors, outputs`` in which the built function takes its arguments
    (graph.py:91-102).
    """

    def __init__(self, name, ops, inputs, weights, const_scalars, const_tensors):
        self.name = name
        self.ops = list(ops)
        self.inputs = list(inputs)
        self.weights = list(weights)
        self.const_scalars = list(const_scalars)
        self.const_tensors = list(const_tensors)
        declared = set(id(t) for t in self.inputs + self.weights + self.const_tensors)
        for op in self.all_ops:
            if isinstance(op, te.PlaceholderOp) and id(op.output(0)) not in declared:
                raise ValueError(
                    "placeholder %s feeds layer %s but is not listed in inputs / weights / const_tensors"
                    % (op.name, name)
                )

    @property
    def all_ops(self):
        """All ops of the layer in post order (producers first), placeholders included."""
        seen, order = set(), []

        def visit(op):
            if id(op) in seen:
                return
            seen.add(id(op))
            for t in op.input_tensors:
                visit(t.op)
            order.append(op)

        for op in self.ops:
            visit(op)
        return order

    @property
    def num_inputs(self):
        return len(self.inputs)

    @property
    def schedule_tensors(self):
        outs = [op.output(0) for op in self.ops]
        return [*self.inputs, *self.weights, *self.const_scalars, *self.const_tensors, *outs]

    @property
    def feed_graph(self):
        """op -> list of consumer ops."""
        feed = {}
        for op in self.all_ops:
            feed.setdefault(op, [])
            for t in op.input_tensors:
                feed.setdefault(t.op, []).append(op)
        return feed

    @property
    def fingerprint(self):
        parts = []
        for op in self.all_ops:
            kind = getattr(op, "kind", "placeholder")
            attrs = getattr(op, "attrs", None)
            tail = (":" + ",".join("%s=%s" % kv for kv in sorted(attrs.items()))) if attrs else ""
            parts.append("%s:%s:%s:%s%s" % (op.name, kind, list(op.output(0).shape), op.output(0).dtype, tail))
        return "|".join(parts)

    def __str__(self):
        ops = self.all_ops
        ret = "====== Layer(%s) ======\n%d ops in this layer.\ninputs:\n" % (self.name, len(ops))
        for t in self.inputs:
            ret += str(t) + "\n"
        ret += "weights:\n"
        for t in self.weights:
            ret += str(t) + "\n"
        ret += "---------------------------------\n"
        ret += " ".join(op.name for op in ops if isinstance(op, te.ComputeOp))
        return ret

    __repr__ = __str__


def layer(ops, inputs=None, weights=None, const_scalars=None, const_tensors=None, requires_grad=False,
          name="layer"):
    """Make a layer from its output op(s); same signature as the reference's ``ac.layer``."""
    if not isinstance(ops, (list, tuple)):
        ops = [ops]
    if len(ops) == 0:
        raise ValueError("a layer needs at least one output op")
    ops = [o.op if isinstance(o, te.Tensor) else o for o in ops]
    return Layer(name, ops, inputs or [], weights or [], const_scalars or [], const_tensors or [])
