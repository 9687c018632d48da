"""Chain descriptors and the "tensorize" step that turns a described chain into a kernel
choice (reference: python/ditto/auto_tensorize/hyper_fusion.py:21-302,
src/auto_tensorize/hyper_fusion.cc:24-216, 586-607, 1494-1603).

In the reference ``tensorize_cuda`` returns a ``te.Schedule`` that TVM then lowers; here it
returns a ``ChainSchedule``: the recognised chain (which contraction pair, which inter-path
op, which epilogue, shapes and dtypes) that ``ditto_amd.build`` binds to one hand-written
gfx950 kernel through the C ABI.  The 13-integer ``CUDATensorizeParam`` is accepted for
source compatibility; the tile actually used comes from the library's per-shape table
(``ditto_bmm_chain_select_tile``), which replaces the reference's parameter search.
"""
from dataclasses import dataclass
from typing import Dict, List

from .. import te
from ..auto_compute.graph import Layer
from ..hardware import HardwareParam


@dataclass
class FusionChoice:
    first_op: te.Operation
    second_op: te.Operation
    ordered_iters: List[te.IterVar]
    attach_pos: int
    # filled by build_fusion_choice (hyper_fusion.cc:2030-2078): the split factor and the index (position
    # among the second op's spatial-then-reduce iteration variables) of every fused outer loop
    secondOpOuterTilingFactors: List[int] = None
    secondOpOuterIndices: List[int] = None

    def __str__(self):
        return "FusionChoice(axis=%s, pos=%d)" % (self.ordered_iters, self.attach_pos)


def fusion_choice(first_op, second_op, ordered_iters, attach_pos):
    return FusionChoice(first_op, second_op, list(ordered_iters), int(attach_pos))


_DTYPE_BYTES = {"float32": 4, "float64": 8, "float16": 2, "bfloat16": 2, "int16": 2, "int32": 4, "int64": 8, "int8": 1}


def build_fusion_choice(sfs, hw_param=None, dtype="float32", simple_mode=-1):
    """The fusion choice for the two contractions of a serial fusion state whose tensorize axes
    are registered (reference: hyper_fusion.py:271-295, hyper_fusion.cc:1974-2079).

    The reference searches over tilings and loop orders of both ops with a cache-level cost model
    (``simple_mode`` 0: full search, -1: pruned search, 1: the identity order) and returns the
    second op's loops in the winning order followed by its tensorized loops, with ``attach_pos``
    = the last loop the first op is computed under.  The gfx950 kernels fix tiling and order
    themselves, so every mode returns the order all of the reference's own drivers choose by hand
    (bmm_bmm_cuda.py:176 ``[b, m, n, rlo, mi, ni, rli], 3``; conv3x3_conv1x1_cuda.py:211
    ``[b, no, p, mo, rlo, mi, ni, rli], 4``; conv1x1_conv3x3_cuda.py:228
    ``[b, no, p, mo, rlo, mi, ni, rr, rs, rli], 4``): the spatial loops that are not tensorized,
    the outermost reduce loop that is not tensorized, the tensorized spatial loops, the remaining
    reduce loops, the tensorized reduce loop; the first op is attached under that outermost
    reduce loop."""
    if not getattr(sfs, "tensorize_axes", None):
        raise ValueError("register the tensorize axes first (SerialFusionState.register_tensorize_axes)")
    if dtype not in _DTYPE_BYTES:
        raise ValueError("unknown dtype %s" % dtype)
    if simple_mode not in (-1, 0, 1):
        raise ValueError("simple_mode must be 1 (a pick without search), 0 (full search) or -1 (pruned search)")
    op1, op2 = sfs.first_op, sfs.second_op
    tens = sfs.tensorize_axes.get(op2, [])
    if not tens:
        raise ValueError("no tensorize axes registered for the second contraction %s" % op2.name)

    def is_tens(iv):
        return any(iv is t for t in tens)

    spatial_nt = [iv for iv in op2.axis if not is_tens(iv)]
    reduce_nt = [iv for iv in op2.reduce_axis if not is_tens(iv)]
    ordered = (spatial_nt + reduce_nt[:1] + [iv for iv in op2.axis if is_tens(iv)] + reduce_nt[1:]
               + [iv for iv in op2.reduce_axis if is_tens(iv)])
    attach_pos = len(spatial_nt) + len(reduce_nt[:1]) - 1
    if attach_pos < 0:
        raise ValueError("no loop of %s is left to attach the first contraction under" % op2.name)
    all_iters = op2.axis + op2.reduce_axis
    outer = ordered[: attach_pos + 1]
    return FusionChoice(op1, op2, ordered, attach_pos, [1] * len(outer),
                        [next(i for i, v in enumerate(all_iters) if v is iv) for iv in outer])


@dataclass
class MatchInfo:
    axis: List[te.IterVar]
    intrin: object
    impl: str = ""

    def __str__(self):
        return "MatchInfo(axis=%s, intrin=%s)" % (self.axis, self.intrin)


def match_info(axis, intrin, impl=""):
    return MatchInfo(list(axis), intrin, impl)


class TensorizeHyperFusionState:
    """Partition of the layer DAG around the two contractions: prologues of each, the single
    path between them, and the epilogue (hyper_fusion.cc:51-216)."""

    def __init__(self, layer: Layer, fuse_choice: FusionChoice, match_info: Dict[te.Operation, MatchInfo]):
        self.layer = layer
        self.fuse_choice = fuse_choice
        self.match_info = dict(match_info or {})
        self.first_op = fuse_choice.first_op
        self.second_op = fuse_choice.second_op
        if not fuse_choice.attach_pos < len(fuse_choice.ordered_iters):
            raise ValueError("attach_pos %d out of range of %d ordered iters"
                             % (fuse_choice.attach_pos, len(fuse_choice.ordered_iters)))
        self.fused_spatial_outer_iters, self.fused_reduce_outer_iters = [], []
        for iv in fuse_choice.ordered_iters[: fuse_choice.attach_pos + 1]:
            if iv.iter_type == te.DATA_PAR:
                self.fused_spatial_outer_iters.append(iv)
            elif iv.iter_type == te.COMM_REDUCE:
                self.fused_reduce_outer_iters.append(iv)
            else:
                raise ValueError("Unexpected iter_type %s." % iv.iter_type)
        self.first_op_prologue, self.second_op_prologue = [], []
        self.inter_path, self.epilogue = [], []
        if len(layer.ops) != 1:
            raise ValueError("a fused chain has exactly one output op, got %d" % len(layer.ops))

        prefix = {}
        found = {"first": False, "second": False}

        def helper(op):
            if not isinstance(op, te.ComputeOp):
                return False, False
            if op in prefix or (op is self.first_op and found["first"]) or (op is self.second_op and found["second"]):
                raise ValueError("The same op %s is visited multiple times.\n"
                                 "The given layer is not a tree structure." % op.name)
            met_first = met_second = False
            if op is self.first_op:
                for inp in op.input_tensors:
                    f, s = helper(inp.op)
                    if f or s or found["first"] or found["second"]:
                        raise ValueError("the first contraction must not consume a contraction")
                    if inp.op in prefix:
                        self.first_op_prologue.append(prefix[inp.op])
                found["first"] = True
                met_first = True
            elif op is self.second_op:
                first_in_producer = False
                for inp in op.input_tensors:
                    f, s = helper(inp.op)
                    if s or found["second"]:
                        raise ValueError("the second contraction appears twice")
                    first_in_producer |= f
                    if inp.op in prefix:
                        if f:
                            if self.inter_path:
                                raise ValueError("Multiple paths from first op to second op.")
                            self.inter_path = prefix[inp.op]
                        else:
                            self.second_op_prologue.append(prefix[inp.op])
                if not first_in_producer:
                    raise ValueError("First op is not the producer of second op.")
                found["second"] = True
                met_second = True
            else:
                chain = []
                for inp in op.input_tensors:
                    f, s = helper(inp.op)
                    met_first |= f
                    met_second |= s
                    chain.extend(prefix.get(inp.op, []))
                prefix[op] = chain + [op]
            return met_first, met_second

        helper(layer.ops[0])
        if layer.ops[0] in prefix:
            self.epilogue = prefix[layer.ops[0]]
        if not (found["first"] and found["second"]):
            raise ValueError("the layer does not contain both contraction ops of the fusion choice")
        if self.first_op not in match_info or self.second_op not in match_info:
            raise ValueError("match_info must cover both contraction ops")
        self.tensorize_iters = {op: mi.axis for op, mi in match_info.items()}
        self.tensorize_intrinsics = {op: mi.intrin for op, mi in match_info.items()}
        self.tensorize_impl = {op: mi.impl for op, mi in match_info.items()}

    def __str__(self):
        return "TensorizeHyperFusionState(layer=%s)" % self.layer.name

    def summary(self, verbose=False):
        ret = "TensorizeHyperFusionState Summary:\n==================================\n"
        ret += "First op: %s\nSecond op: %s\n" % (self.first_op.name, self.second_op.name)
        if verbose:
            line = "----------------------------------\n"
            ret += line + "First op prologue:\n" + line
            for v in self.first_op_prologue:
                ret += "[" + " ".join(o.name for o in v) + " ]\n"
            ret += line + "Second op prologue:\n" + line
            for v in self.second_op_prologue:
                ret += "[" + " ".join(o.name for o in v) + " ]\n"
            ret += line + "Inter Path:\n[" + " ".join(o.name for o in self.inter_path) + " ]\n"
            ret += line + "Epilogue:\n[" + " ".join(o.name for o in self.epilogue) + " ]\n"
            ret += line + "Fused outer spatial iters: %s\n" % self.fused_spatial_outer_iters
            ret += "Fused outer reduce iters: %s\n" % self.fused_reduce_outer_iters
        ret += "==================================\n"
        return ret


def tensorize_hyper_fusion_state(layer, fuse_choice, match_info):
    return TensorizeHyperFusionState(layer, fuse_choice, match_info)


@dataclass
class CUDATensorizeParam:
    warp_size: int = 32
    ty_size: int = 4
    tz_size: int = 2
    input_vector_len: int = 4
    serial_y: int = 2
    serial_z: int = 1
    block_rx: int = 4
    block_ry: int = 1
    block_rz: int = 4
    warp_rx: int = 1
    warp_ry: int = 4
    warp_rz: int = 1
    unroll_steps: int = 1500

    def to_json(self):
        # the same eleven keys the reference serialises (hyper_fusion.py:143-156)
        keys = ["warp_size", "ty_size", "tz_size", "input_vector_len", "serial_y", "serial_z", "block_rx",
                "warp_rx", "block_ry", "warp_ry", "unroll_steps"]
        return {k: getattr(self, k) for k in keys}

    def __str__(self):
        return str(self.to_json())


def cuda_tensorize_param(warp_size=32, ty_size=4, tz_size=2, input_vector_len=4, serial_y=2, serial_z=1,
                         block_rx=4, block_ry=1, block_rz=4, warp_rx=1, warp_ry=4, warp_rz=1, unroll_steps=1500):
    return CUDATensorizeParam(warp_size, ty_size, tz_size, input_vector_len, serial_y, serial_z, block_rx,
                              block_ry, block_rz, warp_rx, warp_ry, warp_rz, unroll_steps)


@dataclass
class ChainSchedule:
    """What ``tensorize_cuda`` / ``tensorize_hip`` returns: the recognised chain."""
    layer: Layer
    state: TensorizeHyperFusionState
    kind: str            # "bmm_chain" | "conv_chain"
    inter_op: str        # "cast" | "relu" | "softmax"
    in_dtype: str
    acc_dtype: str
    out_dtype: str
    dims: dict
    softmax_scale: float = 1.0
    relu_out: bool = False
    hw_param: HardwareParam = None
    tensorize_param: CUDATensorizeParam = None
    requant_scale: float = 1.0       # inter_op "requant": the scale of every column ...
    scale_tensor: bool = False       # ... unless a float32 scale[L] placeholder follows A, B, C
    tile_variant: int = 0            # 0: the library's per-shape table; else the variant id to force
    target: str = "hip"              # "cpu": from tensorize_cpu / FusionContext.run, built with target "llvm"


def _kinds(ops):
    return [op.kind for op in ops]


def _recognise(layer, state):
    first, second = state.first_op, state.second_op
    if first.kind != "contract" or second.kind != "contract":
        raise ValueError("The fusion and tensorize decisions are not valid.")
    inter = _kinds(state.inter_path)
    epi = _kinds(state.epilogue)
    out_t = layer.ops[0].output(0)
    if first.attrs.get("conv"):
        # conv -> (cast|relu) -> pad -> conv -> (cast|relu)
        if len(inter) != 2 or inter[0] not in ("cast", "relu") or inter[1] != "pad":
            raise ValueError("unsupported inter path %s for a conv chain" % inter)
        if epi not in (["unpack_cast"], ["relu_cast"]):
            raise ValueError("unsupported epilogue %s for a conv chain" % epi)
        img = first.input_tensors[0].op.input_tensors[0]  # pad1 <- Img
        w1, w2 = first.input_tensors[1], second.input_tensors[1]
        N, C0, H, W = img.shape
        C1, _, R1, S1 = w1.shape
        C2, _, R2, S2 = w2.shape
        dims = dict(N=N, C0=C0, H=H, W=W, C1=C1, R1=R1, S1=S1, pad1=first.attrs["padding"],
                    stride1=first.attrs["stride"], C2=C2, R2=R2, S2=S2, pad2=second.attrs["padding"],
                    stride2=second.attrs["stride"], groups1=first.attrs.get("groups", 1))
        return dict(kind="conv_chain", inter_op=inter[0], dims=dims, relu_out=epi == ["relu_cast"],
                    in_dtype=img.dtype, acc_dtype=first.output(0).dtype, out_dtype=out_t.dtype, softmax_scale=1.0)
    # batched GEMM chain: dims from the layer's input placeholders
    A, B, C = layer.inputs[:3] if len(layer.inputs) >= 3 else (layer.inputs + layer.weights)[:3]
    batch, M, K = A.shape
    L, N = B.shape[2], C.shape[2]
    dims = dict(batch=batch, M=M, N=N, K=K, L=L)
    if inter == ["exp"]:
        pro = [k for chain in state.second_op_prologue for k in _kinds(chain)]
        pads = [op for chain in state.second_op_prologue for op in chain if op.kind == "pad"]
        if pro != ["pad"] or pads[0].attrs.get("pad_value") != 1 or epi != ["unpack_divide"]:
            raise ValueError("an exp inter path needs the ones-column operand and the divide epilogue "
                             "(got prologue %s, epilogue %s)" % (pro, epi))
        return dict(kind="bmm_chain", inter_op="softmax", dims=dims, relu_out=False, in_dtype=A.dtype,
                    acc_dtype=first.output(0).dtype, out_dtype=out_t.dtype,
                    softmax_scale=state.inter_path[0].attrs.get("scale", 1.0))
    relu_out = epi == ["relu_cast"]  # an activation layer fused into the chain (chimera.graph_fusion)
    if inter == ["requant"] and epi == ["unpack_cast"]:
        req = state.inter_path[0]
        if A.dtype != "int8" or first.output(0).dtype != "int32":
            raise ValueError("a requantised middle result belongs to the int8 / int32 chain")
        has_tensor = len(req.input_tensors) == 2
        return dict(kind="bmm_chain", inter_op="requant", dims=dims, relu_out=False, in_dtype=A.dtype,
                    acc_dtype="int32", out_dtype=out_t.dtype, softmax_scale=1.0,
                    requant_scale=1.0 if has_tensor else float(req.attrs["scale"]), scale_tensor=has_tensor)
    if inter in (["cast"], ["relu"]) and (epi == ["unpack_cast"] or relu_out):
        if A.dtype == "int8":
            # the reference's own int8 chain (bmm_bmm_cuda.py:114-118, 145-149): astype("int8") of the int32
            # accumulators keeps their low byte, for the middle result and (out_dtype int8) for the output
            if first.output(0).dtype != "int32" or out_t.dtype not in ("int8", "int32") or relu_out:
                raise ValueError("the int8 chain accumulates in int32 and outputs int8 or int32, without an output ReLU")
            return dict(kind="bmm_chain", inter_op=inter[0], dims=dims, relu_out=False, in_dtype=A.dtype,
                        acc_dtype="int32", out_dtype=out_t.dtype, softmax_scale=1.0)
        return dict(kind="bmm_chain", inter_op=inter[0], dims=dims, relu_out=relu_out, in_dtype=A.dtype,
                    acc_dtype=first.output(0).dtype, out_dtype=out_t.dtype, softmax_scale=1.0)
    raise ValueError("The fusion and tensorize decisions are not valid (inter path %s, epilogue %s)." % (inter, epi))


def tensorize_hip(layer, state, hip_param=None, tensorize_param=None, tile_variant=0):
    """Bind a described chain to its gfx950 kernel family.  Raises ``ValueError`` for chains
    the path does not cover, where the reference raises ``TVMError`` from a failed CHECK.
    ``tile_variant`` forces a kernel variant (an id ``select_tile`` reports): the counterpart of
    the explicit ``CUDATensorizeParam`` the reference's callers pass."""
    info = _recognise(layer, state)
    return ChainSchedule(layer=layer, state=state, hw_param=hip_param, tensorize_param=tensorize_param,
                         tile_variant=int(tile_variant), **info)


def tensorize_cuda(layer, state, cuda_param=None, tensorize_param=None):
    """Same entry point and argument list as the reference's (hyper_fusion.py:191-197)."""
    return tensorize_hip(layer, state, cuda_param, tensorize_param)



@dataclass
class CPUTensorizeParam:
    """Loop tiling of the CPU fused nest (hyper_fusion.cc:609-642: per-op tiling factors and loop orders chosen by
    ``buildCPUTensorizeParam``).  The nest of this build has two free factors, the ones the reference's search
    spends its time on: ``m_block``, the rows of the chain one parallel task owns (the tiling of the second
    contraction's outer spatial loop), and ``l_block``, the columns of the intermediate computed at the attach
    position before the second contraction consumes them (the tiling of its outer reduce loop).  ``cost`` is the
    analytic score the candidates are ranked by (seconds of a cache-traffic model; a rank, not a time)."""
    firstOpTilingFactor: tuple = ()
    firstOpLoopOrder: tuple = ()
    secondOpTilingFactor: tuple = ()
    secondOpLoopOrder: tuple = ()
    parallelism: int = 1
    mi: int = 6
    ni1: int = 16
    ni2: int = 16
    m_block: int = 6
    l_block: int = 16
    fusion_level: int = -1
    cost: float = 0.0


def cpu_tensorize_candidates(sfs, fusion_choice, hw_param, dtype, dims=None, mi=6, ni1=16, ni2=16):
    """Every (m_block, l_block) tiling of the fused nest for a GEMM chain of extents ``dims`` = (batch, M, N, K, L),
    ranked by a cache model in the spirit of the reference's (hyper_fusion_cpu.cc:1000-1500: footprint of the
    fused tile against the cache sizes picks the level it lives in, bytes moved across that level over its
    bandwidth price the candidate): per task the first contraction's tile, the panels of B and C it meets and its
    rows of A and F must sit in one cache level; B and C are streamed once per task, so fewer, taller tasks move
    fewer bytes but leave cores idle when there are fewer tasks than cores."""
    if dtype not in _DTYPE_BYTES:
        raise ValueError("unknown dtype %s" % dtype)
    eb = _DTYPE_BYTES[dtype]
    batch, M, N, K, L = dims
    par = max(1, int(getattr(hw_param, "num_groups", 1) or 1))
    caches = list(getattr(hw_param, "cacheSizes", None) or [32 * 16, 32 * 1024, 1024 * 1024, 32 * 1024 * 1024])
    bws = list(getattr(hw_param, "bandwidth", None) or [293.72, 81.72, 38.54, 13.14])
    all2 = sfs.second_op.axis + sfs.second_op.reduce_axis
    order2 = tuple(next(i for i, v in enumerate(all2) if v is iv) for iv in fusion_choice.ordered_iters)
    n1 = len(sfs.first_op.axis + sfs.first_op.reduce_axis)
    out = []
    mbs = sorted({min(-(-M // mi) * mi, mi * f) for f in (1, 2, 4, 8, 16, 32, 64)})
    lbs = sorted({min(-(-L // ni1) * ni1, ni1 * f) for f in (1, 2, 4, 8, 16, 32, 64, 1 << 20)})
    for mb in mbs:
        for lb in lbs:
            foot = (mb * lb + K * lb + lb * N + mb * K + mb * N) * eb
            level = next((i for i, c in enumerate(caches) if foot <= c), len(caches) - 1)
            tasks = batch * -(-M // mb)
            rounds = -(-tasks // par)
            moved = (K * L + L * N + mb * (K + N)) * eb          # per task, across the level the tile lives in
            flops = 2.0 * mb * L * (K + N)
            per_task = moved / (bws[min(level + 1, len(bws) - 1)] * 1e9) + flops / (32.0 * 2.5e9)
            p = CPUTensorizeParam(firstOpTilingFactor=(1,) * n1, firstOpLoopOrder=tuple(range(n1)),
                                  secondOpTilingFactor=(1, mb // mi, 1, max(1, lb // ni1)) + (1,) * max(0, len(all2) - 4),
                                  secondOpLoopOrder=order2, parallelism=par, mi=mi, ni1=ni1, ni2=ni2, m_block=mb,
                                  l_block=lb, fusion_level=level, cost=rounds * per_task)
            out.append(p)
    out.sort(key=lambda p: (p.cost, p.m_block, p.l_block))
    return out


def build_cpu_tensorize_param(sfs, fusion_choice, hw_param, dtype, dims=None):
    """The best-ranked tiling (reference: hyper_fusion.py:297-302).  Without ``dims`` (a chain whose extents are not
    known here) the identity tiling in the loop order of ``fusion_choice``."""
    if dtype not in _DTYPE_BYTES:
        raise ValueError("unknown dtype %s" % dtype)
    if dims is not None:
        return cpu_tensorize_candidates(sfs, fusion_choice, hw_param, dtype, dims)[0]
    op1, op2 = sfs.first_op, sfs.second_op
    n1, n2 = len(op1.axis + op1.reduce_axis), len(op2.axis + op2.reduce_axis)
    all2 = op2.axis + op2.reduce_axis
    order2 = tuple(next(i for i, v in enumerate(all2) if v is iv) for iv in fusion_choice.ordered_iters)
    return CPUTensorizeParam((1,) * n1, tuple(range(n1)), (1,) * n2, order2,
                             int(getattr(hw_param, "num_groups", 1) or 1))


def tensorize_cpu(layer, state, cpu_param=None, tensorize_param=None):
    """Bind a described GEMM chain to the CPU fused nest (reference: hyper_fusion.py:262-268,
    hyper_fusion_cpu.cc:1553-1614): the chain is recognised exactly as for the GPU flow (descriptor errors
    surface the same way) and the ``ChainSchedule`` comes back marked for the CPU target, carrying the tiling
    (``tensorize_param``: a ``CPUTensorizeParam``; None: the nest's default) and the micro-kernel sources of the
    state's match infos.  ``ditto_amd.build(sch, tensors, "llvm")`` turns it into a callable over host tensors.
    fp32 / fp64 GEMM chains (cast, relu, softmax between the contractions) only, as in the reference."""
    sch = tensorize_hip(layer, state, cpu_param, None)
    if sch.kind != "bmm_chain" or sch.in_dtype not in ("float32", "float64"):
        raise ValueError("the CPU target runs fp32 / fp64 GEMM chains (got %s, %s)" % (sch.kind, sch.in_dtype))
    if tensorize_param is not None and not isinstance(tensorize_param, CPUTensorizeParam):
        raise TypeError("tensorize_param must be a CPUTensorizeParam")
    sch.tensorize_param = tensorize_param
    sch.target = "cpu"
    return sch
