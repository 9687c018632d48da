"""``build``: from a ``ChainSchedule`` to a callable with the reference's calling convention.

Replaces ``func = tvm.build(sch, layer.schedule_tensors, "cuda")`` followed by
``func(*inputs, *outputs)`` and ``func.time_evaluator(func.entry_name, ctx, min_repeat_ms=600)``
(benchmark/chimera/cuda/bmm_softmax_bmm_cuda.py:23-42, 239, 256).
"""
from . import chain
from .auto_tensorize.hyper_fusion import ChainSchedule


class TimeResult:
    def __init__(self, results):
        self.results = tuple(results)
        self.mean = sum(results) / len(results)

    def __repr__(self):
        return "TimeResult(mean=%.3e s, repeats=%d)" % (self.mean, len(self.results))


class ChainFunction:
    """The built chain.  Called as ``f(*inputs, *outputs)`` with torch tensors on a HIP device,
    in ``layer.schedule_tensors`` order; the output is written in place (destination passing)
    and the call returns without synchronising."""

    entry_name = "default_function"

    def __init__(self, sch: ChainSchedule, tensors=None, target="hip"):
        if not isinstance(sch, ChainSchedule):
            raise TypeError("build expects the ChainSchedule returned by tensorize_cuda / tensorize_hip")
        if target not in ("hip", "rocm", "cuda"):
            raise ValueError("the fused chains are built for HIP devices only (target %r)" % target)
        self.sch = sch
        self.tensors = list(tensors) if tensors is not None else sch.layer.schedule_tensors
        self.target = "hip"

    def _check_args(self, args):
        if len(args) != len(self.tensors):
            raise ValueError("expected %d tensors (inputs then outputs), got %d" % (len(self.tensors), len(args)))
        for a, t in zip(args, self.tensors):
            if tuple(a.shape) != tuple(t.shape):
                raise ValueError("argument for %s has shape %s, expected %s" % (t.name, tuple(a.shape), t.shape))

    def __call__(self, *args):
        self._check_args(args)
        s = self.sch
        if s.kind == "bmm_chain":
            A, B, C, F = args
            chain.run_bmm_chain(A, B, C, F, s.inter_op, s.softmax_scale)
        elif s.kind == "conv_chain":
            X, W1, W2, Y = args
            d = s.dims
            chain.run_conv_chain(X, W1, W2, Y, d["pad1"], d["stride1"], d["pad2"], d["stride2"], s.inter_op,
                                 s.relu_out, groups1=d.get("groups1", 1))
        else:
            raise NotImplementedError("no kernel family for chain kind %r" % s.kind)

    def time_evaluator(self, func_name=None, ctx=None, number=1, repeat=1, min_repeat_ms=0):
        """Mean seconds per call measured with HIP events on the current stream: ``repeat``
        measurements of ``number`` calls each, ``number`` grown until one measurement lasts
        ``min_repeat_ms`` (TVM's rule, used by the reference with ``min_repeat_ms=600``)."""
        import torch

        def evaluator(*args):
            self(*args)
            torch.cuda.synchronize()
            n = max(1, int(number))
            results = []
            for _ in range(max(1, int(repeat))):
                while True:
                    e0 = torch.cuda.Event(enable_timing=True)
                    e1 = torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(n):
                        self(*args)
                    e1.record()
                    e1.synchronize()
                    ms = e0.elapsed_time(e1)
                    if ms >= min_repeat_ms or n >= (1 << 24):
                        break
                    n = max(n + 1, int(n * max(1.5, min_repeat_ms / max(ms, 1e-3) * 1.05)))
                results.append(ms * 1e-3 / n)
            return TimeResult(results)

        return evaluator


class AttentionFunction:
    """The built ``multi_head_attention_mma_layer``: ``f(query_key_value, out)`` runs the fused
    BMM -> softmax -> BMM chain over the per-head views of the packed projection."""

    entry_name = "default_function"

    def __init__(self, sch, tensors=None, target="hip"):
        if target not in ("hip", "rocm", "cuda"):
            raise ValueError("the fused chains are built for HIP devices only (target %r)" % target)
        self.sch = sch
        self.tensors = list(tensors) if tensors is not None else sch.layer.schedule_tensors

    def __call__(self, query_key_value, out):
        for a, t in zip((query_key_value, out), self.tensors):
            if tuple(a.shape) != tuple(t.shape):
                raise ValueError("argument for %s has shape %s, expected %s" % (t.name, tuple(a.shape), t.shape))
        self.sch.module.forward(query_key_value, out, tile_variant=self.sch.tile_variant)


def build(sch, tensors=None, target="hip", name="default_function"):
    from .auto_schedule.schedulers.chimera_integrate import AttentionSchedule

    if isinstance(sch, AttentionSchedule):
        return AttentionFunction(sch, tensors, target)
    return ChainFunction(sch, tensors, target)
