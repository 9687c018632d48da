"""Operator pattern classification (reference: src/auto_tensorize/pattern.cc:13-100,
include/auto_tensorize/config.h:7 for SUBSTANTIAL)."""
from .. import te

SUBSTANTIAL = 16

PATTERN_CUBIC = "PATTERN_CUBIC"
PATTERN_ALLRED = "PATTERN_ALLRED"
PATTERN_SHUFFLE = "PATTERN_SHUFFLE"
PATTERN_LOCAL = "PATTERN_LOCAL"


def _uses(op, input_idx, iv):
    return any(v is iv for v in op.accesses[input_idx][1])


def IsCubic(op, substantial=SUBSTANTIAL):
    """A contraction: at least two inputs, every input owns a spatial iteration variable of
    extent >= ``substantial`` that no other input uses, and some reduce variable of extent
    >= ``substantial`` is used by all inputs."""
    if not isinstance(op, te.ComputeOp):
        return False
    n_in = len(op.accesses)
    if n_in < 2:
        return False
    owners = set()
    for iv in op.axis:
        if iv.extent < substantial:
            continue
        users = [i for i in range(n_in) if _uses(op, i, iv)]
        if len(users) == 1:
            owners.add(users[0])
    is_outer = len(owners) == n_in
    is_inner = any(iv.extent >= substantial and all(_uses(op, i, iv) for i in range(n_in))
                   for iv in op.reduce_axis)
    return (is_outer and is_inner) or ("PATTERN_CUBIC" in op.tag)


def IsAllred(op, substantial=SUBSTANTIAL):
    """A reduction over one input (e.g. a row sum)."""
    if not isinstance(op, te.ComputeOp) or len(op.accesses) != 1:
        return False
    return any(iv.extent >= substantial for iv in op.reduce_axis) or ("PATTERN_ALLRED" in op.tag)


def IsShuffle(op):
    """Pure data movement whose output indices are not the input indices (pack, pad, transpose)."""
    return isinstance(op, te.ComputeOp) and op.kind in ("pack", "pad", "unpack", "transpose") and not op.reduce_axis


def IsLocal(op):
    """Elementwise: every input is indexed exactly by the output's iteration variables."""
    if not isinstance(op, te.ComputeOp) or op.reduce_axis:
        return False
    return not IsShuffle(op)


def GetOpPattern(op):
    if IsCubic(op):
        return PATTERN_CUBIC
    if IsAllred(op):
        return PATTERN_ALLRED
    if IsShuffle(op):
        return PATTERN_SHUFFLE
    return PATTERN_LOCAL
