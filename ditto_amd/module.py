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
            raise ValueError("a schedule for the CPU target is built with target \"llvm\" (ditto_amd.build), and a "
                             "schedule for HIP devices with \"hip\": got schedule %r, target %r" % (sch.target, target))
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
        if self.sch.kind == "conv_chain" and args[0].dim() == 5:
            return  # the reference's packed placeholders: checked in _call_packed
        for a, t in zip(args, self.tensors):
            if tuple(a.shape) != tuple(t.shape):
                raise ValueError("argument for %s has shape %s, expected %s" % (t.name, tuple(a.shape), t.shape))

    def _call_packed(self, img_p, w1_p, w2_p, out_p):
        """The reference's calling convention for conv chains: packed, pre-padded tensors
        (conv3x3_conv1x1_cuda.py:90-105; ``ditto_amd.layout``).  The padded image is unpacked to NCHW and the first
        convolution runs over it without padding (the border is the caller's, as in the reference); the weights are
        unpacked once per pair of weight tensors (kept like ``specialize`` keeps its weights: by identity and
        version); the result is packed into ``out_p``.  Stride 1."""
        from . import layout

        d = self.sch.dims
        if d["stride1"] != 1 or d["stride2"] != 1:
            raise NotImplementedError("packed placeholders are taken for stride 1 chains")
        N, C0, H, W = d["N"], d["C0"], d["H"], d["W"]
        pad1 = d["pad1"]
        Q = (W + 2 * pad1 - d["S1"]) + 1 + 2 * d["pad2"] - d["S2"] + 1
        P = (H + 2 * pad1 - d["R1"]) + 1 + 2 * d["pad2"] - d["R2"] + 1
        if tuple(img_p.shape[:3]) != (N, C0 // 16, H + 2 * pad1) or img_p.shape[3] < W + 2 * pad1 or C0 % 16:
            raise ValueError("packed image must be [%d, %d, %d, >= %d, 16], got %s"
                             % (N, C0 // 16, H + 2 * pad1, W + 2 * pad1, tuple(img_p.shape)))
        x = layout.unpack_image(img_p, W + 2 * pad1)
        cache = getattr(self, "_packed_weights", None)
        if not (cache and cache[0] is w1_p and cache[1] is w2_p and cache[2] == (w1_p._version, w2_p._version)):
            cache = (w1_p, w2_p, (w1_p._version, w2_p._version), layout.unpack_weight(w1_p), layout.unpack_weight(w2_p))
            self._packed_weights = cache
        w1, w2 = cache[3], cache[4]
        want1 = (d["C1"], C0 // d.get("groups1", 1), d["R1"], d["S1"])
        if tuple(w1.shape) != want1 or tuple(w2.shape) != (d["C2"], d["C1"], d["R2"], d["S2"]):
            raise ValueError("packed weights do not match the chain: %s, %s" % (tuple(w1_p.shape), tuple(w2_p.shape)))
        f = getattr(self, "_packed_fn", None)
        if f is None:  # the same chain with the first padding taken out of the kernel's hands
            import copy

            sch = copy.copy(self.sch)
            sch.dims = dict(d, H=H + 2 * pad1, W=W + 2 * pad1, pad1=0)
            f = self._packed_fn = ChainFunction(sch, [None] * 4, self.target, self.tile_variant)
            f._check_args = lambda args: None
        y = torch.empty((N, d["C2"], P, Q), device=x.device, dtype=out_p.dtype)
        f(x, w1, w2, y)
        layout.pack_output_into(y, out_p)

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
            if X.dim() == 5:
                return self._call_packed(X, W1, W2, Y)
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


class CpuChainFunction:
    """A GEMM chain built for the CPU target: ``f(A, B, C, F)`` over host tensors (torch CPU tensors or numpy
    arrays, fp32 / fp64, rows contiguous), blocking like the reference's LLVM-target function.  The fused loop nest
    is ``libditto_chain_cpu.so`` (``csrc/cpu/chain_cpu.cpp``); its tiling is the schedule's ``CPUTensorizeParam``
    and its full register tiles run on the micro-kernels compiled from the sources ``cpu_intrin`` generated, where
    the schedule's match infos carry any (reference flow: benchmark/chimera/cpu/bmm_bmm_cpu.py:118-276)."""

    entry_name = "default_function"

    def __init__(self, sch, tensors=None, name="default_function"):
        from . import _cpu_lib
        from .auto_tensorize.hyper_fusion import CPUTensorizeParam

        if sch.kind != "bmm_chain" or sch.in_dtype not in ("float32", "float64"):
            raise NotImplementedError("the CPU target runs fp32 / fp64 GEMM chains (got %s, %s)" % (sch.kind, sch.in_dtype))
        if sch.inter_op not in ("cast", "relu", "softmax"):
            raise NotImplementedError("no CPU nest for inter op %r" % sch.inter_op)
        self.sch = sch
        self.tensors = list(tensors) if tensors is not None else sch.layer.schedule_tensors
        self.target = "llvm"
        self.entry_name = name
        self._lib = _cpu_lib.load()
        p = sch.tensorize_param if isinstance(sch.tensorize_param, CPUTensorizeParam) else CPUTensorizeParam()
        d = sch.dims
        self.param = p
        self._update = [None, None]
        infos = getattr(sch.state, "match_info", {}) or {}
        mi, ni1, ni2 = p.mi, p.ni1, p.ni2
        for slot, op in enumerate((sch.state.first_op, sch.state.second_op)):
            m = infos.get(op)
            if m is not None and m.impl:
                self._update[slot] = _cpu_lib.compile_kernel(m.impl, m.intrin.compute_intrinsic.name)
                ci = m.intrin.compute_intrinsic
                if slot == 0:
                    mi, ni1 = ci.M, ci.N
                else:
                    ni2 = ci.N
        desc = _cpu_lib.CpuChainDesc()
        desc.abi_version = _cpu_lib.ABI_VERSION
        desc.dtype = 2 if sch.in_dtype == "float32" else 5
        desc.inter_op = {"cast": 0, "relu": 1, "softmax": 2}[sch.inter_op]
        desc.relu_out = int(bool(sch.relu_out))
        desc.batch, desc.M, desc.N, desc.K, desc.L = d["batch"], d["M"], d["N"], d["K"], d["L"]
        desc.softmax_scale = float(sch.softmax_scale)
        desc.mi, desc.ni1, desc.ni2 = mi, ni1, ni2
        desc.m_block = max(mi, p.m_block // mi * mi) if p.m_block >= mi else mi
        desc.l_block = max(1, p.l_block)
        desc.threads = max(0, int(p.parallelism if p.parallelism > 1 else 0))
        desc.update1, desc.update2 = self._update
        desc.a_batch_stride, desc.a_row_stride = d["M"] * d["K"], d["K"]
        desc.b_batch_stride, desc.b_row_stride = d["K"] * d["L"], d["L"]
        desc.c_batch_stride, desc.c_row_stride = d["L"] * d["N"], d["N"]
        desc.f_batch_stride, desc.f_row_stride = d["M"] * d["N"], d["N"]
        self._desc = desc

    @staticmethod
    def _host(t):
        import numpy as np

        if isinstance(t, np.ndarray):
            return t
        if t.device.type != "cpu":
            raise ValueError("the CPU target takes host tensors")
        return t.numpy()

    def __call__(self, *args):
        if len(args) != len(self.tensors):
            raise ValueError("expected %d tensors (inputs then outputs), got %d" % (len(self.tensors), len(args)))
        arrs = [self._host(a) for a in args]
        d = self.sch.dims
        want = self.sch.in_dtype
        total = {"A": d["batch"] * d["M"] * d["K"], "B": d["batch"] * d["K"] * d["L"], "C": d["batch"] * d["L"] * d["N"],
                 "F": d["batch"] * d["M"] * d["N"]}
        for a, name in zip(arrs, "ABCF"):
            # the reference's CPU placeholders are the same row-major memory split into micro-kernel tiles
            # ([batch, M / MI, MI, K / KI, KI], bmm_bmm_cpu.py:65-69): any contiguous array of the right size does
            if str(a.dtype) != want or not a.flags["C_CONTIGUOUS"] or a.size != total[name]:
                raise ValueError("%s must be a contiguous %s array of %d elements, got %s %s" % (name, want, total[name],
                                                                                             a.dtype, a.shape))
        import ctypes

        desc = self._desc

        rc = self._lib.ditto_cpu_bmm_chain_run(ctypes.byref(desc), *(a.ctypes.data for a in arrs))
        if rc != 0:
            raise ValueError(self._lib.ditto_cpu_last_error().decode("utf-8", "replace"))

    def time_evaluator(self, func_name=None, ctx=None, number=1, repeat=1, min_repeat_ms=0, f_preproc=""):
        """Mean seconds per call (wall clock; the call is blocking).  ``f_preproc="cache_flush_cpu_non_first_arg"``
        streams a buffer larger than the last-level cache between measurements, as the reference's CPU drivers ask
        of TVM (bmm_bmm_cpu.py:264-266)."""
        import time

        import numpy as np

        flush = np.zeros(64 << 20, dtype=np.uint8) if f_preproc == "cache_flush_cpu_non_first_arg" else None

        def evaluator(*args):
            self(*args)
            results = []
            n = max(1, int(number))
            for _ in range(max(1, int(repeat))):
                while True:
                    if flush is not None:
                        np.add(flush, 1, out=flush)
                    t0 = time.perf_counter()
                    for _ in range(n):
                        self(*args)
                    dt = time.perf_counter() - t0
                    if dt * 1e3 >= min_repeat_ms or n >= (1 << 20):
                        break
                    n = max(n + 1, int(n * max(1.5, min_repeat_ms / max(dt * 1e3, 1e-3) * 1.05)))
                results.append(dt / n)
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
    if target in ("llvm", "cpu", "c"):
        # the reference's CPU flow ends in tvm.build(sch, tensors, name=...) on the LLVM target (bmm_bmm_cpu.py:251)
        if getattr(sch, "target", "hip") != "cpu":
            raise ValueError("target %r needs a schedule from tensorize_cpu / FusionContext.run" % target)
        return CpuChainFunction(sch, tensors, name)
    return ChainFunction(sch, tensors, target, tile_variant)
