"""A light stand-in for the slice of ``tvm.te`` that Ditto's chain builders use.

The reference describes a chain as a DAG of ``tvm.te`` compute ops and hands it to its
C++ scheduler (python/ditto/auto_compute/nn/functional/bmm_chain.py:40-103).  TVM is not
part of this build, so the builders here produce the same DAG *shape* -- placeholders,
compute ops with named spatial / reduce iteration variables, ``op.input_tensors``,
``op.axis``, ``op.reduce_axis``, ``tensor.op`` -- but each op carries a semantic ``kind``
(``"contract"``, ``"exp"``, ``"cast"`` ...) and the list of iteration variables with which it
indexes every input, instead of an expression tree.  That is all the descriptor side
(pattern classification, DAG partition, chain recognition) needs.
"""
import itertools

DATA_PAR = "DataPar"
COMM_REDUCE = "CommReduce"

_uid = itertools.count()


class IterVar:
    """An iteration variable with a static extent (tvm.tir.IterVar stand-in)."""

    def __init__(self, extent, name, iter_type=DATA_PAR):
        self.extent = int(extent)
        self.name = name
        self.iter_type = iter_type
        self._id = next(_uid)

    @property
    def dom(self):
        return (0, self.extent)

    def __repr__(self):
        return "iter_var(%s, range(0, %d), %s)" % (self.name, self.extent, self.iter_type)


def reduce_axis(dom, name="rv"):
    lo, hi = dom
    if lo != 0:
        raise ValueError("reduce_axis must start at 0")
    return IterVar(hi, name, COMM_REDUCE)


class Tensor:
    def __init__(self, op, shape, dtype, name):
        self.op = op
        self.shape = tuple(int(s) for s in shape)
        self.dtype = dtype
        self.name = name

    def astype(self, dtype):
        return self

    def __repr__(self):
        return "Tensor(%s, %s, %s)" % (self.name, list(self.shape), self.dtype)

    def __hash__(self):
        return id(self)

    def __eq__(self, other):
        return self is other


class Operation:
    num_outputs = 1

    def output(self, i):
        if i != 0:
            raise IndexError("ops have one output")
        return self._out

    @property
    def input_tensors(self):
        return list(self._inputs)

    def __hash__(self):
        return id(self)

    def __eq__(self, other):
        return self is other


class PlaceholderOp(Operation):
    def __init__(self, shape, dtype, name):
        self.name = name
        self.tag = ""
        self._inputs = []
        self.axis = []
        self.reduce_axis = []
        self._out = Tensor(self, shape, dtype, name)

    def __repr__(self):
        return "placeholder(%s, %s)" % (self.name, list(self._out.shape))


class ComputeOp(Operation):
    """A compute op.

    kind      what the op computes (see the builders); drives chain recognition
    accesses  for each input tensor, the iteration variables that index it
    attrs     kind-specific attributes (e.g. the padding value, the epsilon of a divide)
    """

    def __init__(self, name, shape, dtype, axis, reduce_axes, accesses, kind, attrs=None, tag=""):
        self.name = name
        self.tag = tag
        self.axis = list(axis)
        self.reduce_axis = list(reduce_axes)
        self.accesses = [(t, list(ivs)) for t, ivs in accesses]
        self._inputs = []
        for t, _ in self.accesses:
            if not any(t is u for u in self._inputs):
                self._inputs.append(t)
        self.kind = kind
        self.attrs = dict(attrs or {})
        if len(shape) != len(self.axis):
            raise ValueError("%s: %d axes for a %d-d output" % (name, len(self.axis), len(shape)))
        self._out = Tensor(self, shape, dtype, name)

    def __repr__(self):
        return "compute(%s, kind=%s, %s)" % (self.name, self.kind, list(self._out.shape))


def placeholder(shape, name="placeholder", dtype="float32"):
    return PlaceholderOp(shape, dtype, name).output(0)


def compute(shape, name, dtype, kind, accesses, axis_names=None, reduce_axes=(), attrs=None, tag=""):
    """Create a compute op and return ``(tensor, axis)``.

    ``accesses`` is a callable ``f(*axis) -> [(input_tensor, [iter vars])]`` so that the
    spatial iteration variables can be created here, named by ``axis_names``.
    """
    names = axis_names or ["ax%d" % i for i in range(len(shape))]
    axis = [IterVar(e, n, DATA_PAR) for e, n in zip(shape, names)]
    acc = accesses(*axis)
    op = ComputeOp(name, shape, dtype, axis, reduce_axes, acc, kind, attrs, tag)
    return op.output(0)
