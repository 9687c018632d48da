"""``SerialFusionState`` and ``validate`` (reference: src/auto_tensorize/state.cc:182-253,
src/auto_tensorize/api.cc:14-31)."""
from .. import te
from .pattern import PATTERN_ALLRED, PATTERN_CUBIC, GetOpPattern


class SerialFusionState:
    """Finds the two contraction ops of a layer; ``first_op`` is the producer side."""

    def __init__(self, layer):
        self.layer = layer
        self.ops = [op for op in layer.all_ops if isinstance(op, te.ComputeOp)]
        self.patterns = {op: GetOpPattern(op) for op in self.ops}
        cubic = [op for op in self.ops if self.patterns[op] == PATTERN_CUBIC]
        if len(cubic) != 2:
            raise ValueError("we only deal with 2 CUBIC ops, but has %d" % len(cubic))
        # all_ops is in producer-first order
        self.first_op, self.second_op = cubic
        self.tensorize_axes = {}

    def IsLinearTopo(self):
        feed = self.layer.feed_graph
        return all(len(feed.get(op, [])) <= 1 for op in self.ops)

    def CountOp(self, pattern):
        return sum(1 for op in self.ops if self.patterns[op] == pattern)

    def register_tensorize_axes(self, axes):
        """``axes``: {op: [iter vars]} handed to the micro-kernel (bmm_bmm_cpu.py:165-170)."""
        self.tensorize_axes.update(axes)


def build_serial_fusion_state(layer):
    return SerialFusionState(layer)


def validate(state):
    """(ok, reason) with the reference's three conditions and messages."""
    if not state.IsLinearTopo():
        return False, "the given layer is not in linear topology."
    n_cubic = state.CountOp(PATTERN_CUBIC)
    if n_cubic not in (1, 2):
        return False, "Ditto expect 1 or 2 cubic operators in the layer."
    if state.CountOp(PATTERN_ALLRED) > 0:
        return False, ("auto_tensorize can't handle all reduce.\n The all reduce ops"
                       "should be eliminated by the frontend.\n Did you forget to use"
                       "Ditto's graph frontend?")
    return True, ""
