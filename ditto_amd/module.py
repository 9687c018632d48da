"""``build``: from a ``ChainSchedule`` to a callable with the reference's calling convention.

Replaces ``func = tvm.build(sch, layer.schedule_tensors, "cuda")`` followed by
``func(*inputs, *outputs)`` and ``func.time_evaluator(func.entry_name, ctx, min_repeat_ms=600)``
(benchmark/chimera/cuda/bmm_softmax_bmm_cuda.py:23-42, 239, 256).
"""
import torch

from . import chain
from .auto_tensorize.hyper_fusion import ChainSchedule

_TORCH = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32, "float64": torch.float64,
          "int8": torch.int8,
          "int32": torch.int32}


class TimeResult:
    def __init__(self, results):
        self.results = tuple(results)
        self.mean = sum(results) / len(results)

    def __repr__(self):
        return "TimeResult(mean=%.3e s, repeats=%d)" % (self.mean, len(self.results))


class ChainFunction:
    """The built chain.  Called as ``f(*inputs, *outputs)`` with torch tensors on a HIP device,
    in ``layer.schedule_tensors`` order; the output is written in place (destination passing)
    and the call returns without synchronising.

    The C-ABI descriptor is filled once per distinct argument layout (shapes, strides, dtypes)
    and reused.  A conv chain that takes a workspace owns one per device, sized by
    ``ditto_conv_chain_workspace_bytes`` at its first call and never replaced, so a HIP graph that
    captured a call keeps a valid pointer; calls of ONE function object on two streams still race
    on it (use ``specialize`` for a second object).  ``specialize(W1, W2)`` returns a function bound
    to fixed weights whose repacking is done once, the counterpart of the reference's drivers being
    handed host-packed weights (conv3x3_conv1x1_cuda.py:99-103): its calls run the fused kernel
    alone for as long as they are given those same weight tensors with unchanged contents.  The function keeps
    the two tensors alive (their addresses cannot be handed to other tensors) and remembers their version
    counters: other tensors, or the same ones after an in-place update, are repacked at that call and become
    the bound weights."""

    entry_name = "default_function"

    def __init__(self, sch: ChainSchedule, tensors=None, target="hip", tile_variant=None):
        if not isinstance(sch, ChainSchedule):
            raise TypeError("build expects the ChainSchedule returned by tensorize_cuda / tensorize_hip")
        if getattr(sch, "target", "hip") != "hip" or target in ("llvm", "cpu", "c"):
            raise NotImplementedError("this build runs the fused chains on HIP devices only: there is no CPU "
                                      "product path (target %r)" % (target if target != "hip" else sch.target))
        if target not in ("hip", "rocm", "cuda"):
            raise ValueError("the fused chains are built for HIP devices only (target %r)" % target)
        self.sch = sch
        self.tensors = list(tensors) if tensors is not None else sch.layer.schedule_tensors
        self.target = "hip"
        self.tile_variant = int(sch.tile_variant if tile_variant is None else tile_variant)
        self._descs = {}        # argument layout -> filled descriptor
        self._workspaces = {}   # device -> uint8 tensor (conv chains)
        self._prepared = None   # (W1, W2, W1._version, W2._version): what the workspace holds the repacked form of

    def _check_args(self, args):
        if len(args) != len(self.tensors):
            raise ValueError("expected %d tensors (inputs then outputs), got %d" % (len(self.tensors), len(args)))
        for a, t in zip(args, self.tensors):
            if tuple(a.shape) != tuple(t.shape):
                raise ValueError("argument for %s has shape %s, expected %s" % (t.name, tuple(a.shape), t.shape))

    @staticmethod
    def _layout(args):
        return tuple((tuple(a.shape), tuple(a.stride()), a.dtype) for a in args)

    def _desc(self, args, make):
        key = self._layout(args)
        d = self._descs.get(key)
        if d is None:
            d = self._descs[key] = make()
        return d

    def _workspace(self, desc, dev):
        ws = self._workspaces.get(dev)
        if ws is None:
            nbytes = chain.conv_chain_workspace_bytes(desc)
            ws = self._workspaces[dev] = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev) if nbytes else False
        return ws

    def _conv_desc(self, X, W1, W2, Y):
        s, d = self.sch, self.sch.dims
        return self._desc((X, W1, W2, Y), lambda: chain.conv_chain_desc(
            X, W1, W2, Y, d["pad1"], d["stride1"], d["pad2"], d["stride2"], s.inter_op, s.relu_out,
            d.get("groups1", 1)))

    def specialize(self, W1, W2):
        """A copy of this conv chain function bound to the weight tensors ``W1``, ``W2``: they are
        repacked once, now, into a workspace of its own."""
        if self.sch.kind != "conv_chain":
            raise ValueError("only conv chains repack weights")
        f = ChainFunction(self.sch, self.tensors, self.target, self.tile_variant)
        xt, _, _, yt = self.tensors
        dt = W1.dtype
        # the descriptor depends on shapes and dtypes only (all four tensors are contiguous)
        X = torch.empty(tuple(xt.shape), device="meta", dtype=dt)
        Y = torch.empty(tuple(yt.shape), device="meta", dtype=_TORCH[yt.dtype])
        d = self.sch.dims
        desc = chain.conv_chain_desc(X, W1, W2, Y, d["pad1"], d["stride1"], d["pad2"], d["stride2"],
                                     self.sch.inter_op, self.sch.relu_out, d.get("groups1", 1))
        ws = f._workspace(desc, W1.device)
        if ws is not False:
            chain.prepare_conv_chain(desc, W1, W2, ws)
            f._prepared = (W1, W2, W1._version, W2._version)
        return f

    def _is_prepared(self, W1, W2):
        p = self._prepared
        if p is None:
            return False

        def same(held, w):  # the held tensor itself, or another view of exactly its memory (views share the counter)
            return held is w or (w.data_ptr() == held.data_ptr() and w.shape == held.shape and w.dtype == held.dtype
                                 and w.device == held.device)

        return same(p[0], W1) and same(p[1], W2) and p[2] == W1._version and p[3] == W2._version

    def __call__(self, *args):
        self._check_args(args)
        s = self.sch
        if s.kind == "bmm_chain":
            aux = None
            if s.scale_tensor:
                A, B, C, aux, F = args
            else:
                A, B, C, F = args
            desc = self._desc((A, B, C, F), lambda: chain.bmm_chain_desc(
                A, B, C, F, s.inter_op, s.softmax_scale, s.requant_scale, self.tile_variant, s.relu_out))
            chain.run_bmm_chain(A, B, C, F, aux=aux, desc=desc)
        elif s.kind == "conv_chain":
            X, W1, W2, Y = args
            desc = self._conv_desc(X, W1, W2, Y)
            ws = self._workspace(desc, X.device)
            prepared = ws is not False and self._is_prepared(W1, W2)
            if ws is not False and self._prepared is not None and not prepared:
                # a specialised function handed other weights (or the bound ones after an in-place update):
                # repack them now; they are the bound weights from here on
                self._prepared = None
                try:
                    chain.prepare_conv_chain(desc, W1, W2, ws)
                    self._prepared = (W1, W2, W1._version, W2._version)
                    prepared = True
                except ValueError:
                    pass  # pointers the prepared form cannot take: the one-call form below decides
            chain.run_conv_chain(X, W1, W2, Y, desc=desc, workspace=ws, prepared=prepared)
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


def build(sch, tensors=None, target="hip", name="default_function", tile_variant=None):
    from .auto_schedule.schedulers.chimera_integrate import AttentionSchedule

    if isinstance(sch, AttentionSchedule):
        return AttentionFunction(sch, tensors, target)
    return ChainFunction(sch, tensors, target, tile_variant)
