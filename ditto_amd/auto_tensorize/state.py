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
        """``axes``: the iteration variables handed to the intrinsics, as one flat list over both
        contractions (state.py:16, bmm_bmm_cpu.py:194-196, test_hyper_fusion.py:866-868) or as
        ``{op: [iter vars]}``.  Every variable must belong to one of the two contractions."""
        if isinstance(axes, dict):
            flat = [(op, iv) for op, ivs in axes.items() for iv in ivs]
        else:
            flat = []
            for iv in axes:
                owner = [op for op in (self.first_op, self.second_op)
                         if any(iv is v for v in op.axis + op.reduce_axis)]
                if not owner:
                    raise ValueError("iter var %s belongs to neither contraction of the layer" % iv.name)
                flat.append((owner[0], iv))
        for op, iv in flat:
            lst = self.tensorize_axes.setdefault(op, [])
            if not any(iv is v for v in lst):
                lst.append(iv)


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


class FusionContext:
    """What ``build_fusion_context`` returns in the reference: the ranked candidate schedules of the CPU fused
    nest (state.py:34-78, hyper_fusion.cc:2182-2247).  The candidates are the (m_block, l_block) tilings of the
    nest ranked by the cache model of ``cpu_tensorize_candidates``; ``mode`` bounds how many are kept ("test": the
    best one, "best": the best five, "survey": all), ``run(i, sch)`` returns candidate ``i`` as a schedule for the
    CPU target, which ``ditto_amd.build(sch, tensors, "llvm")`` builds."""

    def __init__(self, sfs, layer, state, path, hw_param, searchType, mode, dtype):
        from .hyper_fusion import _DTYPE_BYTES, _recognise, cpu_tensorize_candidates

        if searchType not in ("normal", "stochastic"):
            raise ValueError("searchType must be normal or stochastic")
        if mode not in ("survey", "best", "test"):
            raise ValueError("mode must be survey, best or test")
        if dtype not in _DTYPE_BYTES:
            raise ValueError("unknown dtype %s" % dtype)
        self.sfs, self.layer, self.state, self.path = sfs, layer, state, path
        self.hw_param, self.searchType, self.mode, self.dtype = hw_param, searchType, mode, dtype
        self.bytePerEle = _DTYPE_BYTES[dtype]
        info = _recognise(layer, state)
        self.candidates = [None]
        if info["kind"] == "bmm_chain" and info["in_dtype"] in ("float32", "float64"):
            d = info["dims"]
            mi, ni1, ni2 = 6, 16, 16
            infos = getattr(state, "match_info", None) or {}
            m1, m2 = infos.get(sfs.first_op), infos.get(sfs.second_op)
            if m1 is not None and m2 is not None:
                c1, c2 = m1.intrin.compute_intrinsic, m2.intrin.compute_intrinsic
                mi, ni1, ni2 = c1.M, c1.N, c2.N
            cands = cpu_tensorize_candidates(sfs, state.fuse_choice, hw_param, dtype,
                                             (d["batch"], d["M"], d["N"], d["K"], d["L"]), mi, ni1, ni2)
            keep = {"test": 1, "best": 5, "survey": len(cands)}[mode]
            self.candidates = cands[:keep]
        self.size = len(self.candidates)

    def _check(self, i):
        if not 0 <= i < self.size:
            raise IndexError("fusion context holds %d candidate(s)" % self.size)

    def run(self, i, sch=None, verbose=False):
        from .hyper_fusion import tensorize_cpu

        self._check(i)
        out = tensorize_cpu(self.layer, self.state, self.hw_param, self.candidates[i])
        if verbose:
            print(self.state.summary(verbose=True))
            print(self.candidates[i])
        return out

    def getComputation(self, i):
        """Multiply-accumulates of the two contractions."""
        self._check(i)
        total = 0
        for op in (self.sfs.first_op, self.sfs.second_op):
            n = 1
            for iv in op.axis + op.reduce_axis:
                n *= iv.extent
            total += n
        return total

    def getFusionLevel(self, i):
        """Index of the smallest cache level that holds the first contraction's tile under the fused
        loops (one iteration of them), -1 if none does or the hardware record lists no caches."""
        self._check(i)
        fused = self.state.fused_spatial_outer_iters
        op1 = self.sfs.first_op
        elems = 1
        for iv in op1.axis:
            if not any(iv.name == f.name and iv.extent == f.extent for f in fused):
                elems *= iv.extent
        sizes = list(getattr(self.hw_param, "cacheSizes", None) or [])
        for level, cap in enumerate(sizes):
            if elems * self.bytePerEle <= cap:
                return level
        return -1


def build_fusion_context(sfs, layer, state, path, hw_param, searchType="normal", mode="best", dtype="float32"):
    """Same argument list as the reference's (state.py:34-51)."""
    return FusionContext(sfs, layer, state, path, hw_param, searchType, mode, dtype)
