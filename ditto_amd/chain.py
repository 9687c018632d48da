"""Tensor-level entry to the fused chains: torch tensors in, one C-ABI call out.

This is the counterpart of calling the PackedFunc that ``tvm.build`` returns for a
scheduled hyper_fusion layer, ``func(*inputs, *outputs)``
(reference: benchmark/chimera/cuda/bmm_softmax_bmm_cuda.py:256): destination passing,
the caller allocates the output, the call enqueues on the current stream and does not
synchronise.  torch is used only to hold device memory and name the stream.
"""
import ctypes

import torch

from . import _lib

_TORCH_CODES = {
    torch.float16: _lib.F16,
    torch.bfloat16: _lib.BF16,
    torch.float32: _lib.F32,
    torch.float64: _lib.F64,
    torch.int8: _lib.I8,
    torch.int32: _lib.I32,
}

INTER_OPS = {"cast": _lib.INTER_CAST, "relu": _lib.INTER_RELU, "softmax": _lib.INTER_SOFTMAX,
             "requant": _lib.INTER_REQUANT}


def _code(t):
    try:
        return _TORCH_CODES[t.dtype]
    except KeyError:
        raise ValueError("unsupported tensor dtype %s" % t.dtype)


def _raw_stream(index):
    """Handle of torch's current stream on device ``index`` (what ``torch.cuda.current_stream(i).cuda_stream`` returns,
    without building the Stream object)."""
    get = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    return get(index) if get is not None else torch.cuda.current_stream(index).cuda_stream


def _check_device(*tensors):
    dev = tensors[0].device
    if dev.type != "cuda":
        raise ValueError("fused chains run on a HIP device; got a %s tensor" % dev.type)
    for t in tensors:
        if t.device != dev:
            raise ValueError("all tensors of a chain must be on the same device")
    return dev


def _as3d(t, name):
    if t.dim() == 2:
        t = t.unsqueeze(0)
    if t.dim() != 3:
        raise ValueError("%s must be [batch, rows, cols] or [rows, cols]" % name)
    return t


def _split_levels(t, name):
    """[outer, inner, rows, cols] (any strides) -> (3-D view of the first outer entry with the inner
    level as its batch, outer extent, outer stride); 2-D / 3-D tensors have a single level."""
    if t.dim() == 4:
        return t[0], t.shape[0], t.stride(0)
    return _as3d(t, name), 1, 0


def bmm_chain_desc(A, B, C, F, inter_op="cast", softmax_scale=1.0, requant_scale=1.0, tile_variant=0,
                   relu_out=False):
    """Fill a ``ditto_bmm_chain_desc`` from tensors A[b,M,K], B[b,K,L], C[b,L,N], F[b,M,N].

    B may be a transposed view of a ``[b, L, K]`` tensor (stride 1 along K); it is then
    consumed in place (``DITTO_B_LK``).  All four may instead be 4-D ``[outer, inner, rows, cols]``
    views with arbitrary outer / inner strides (e.g. the per-head views of a packed
    ``[batch, seq, 3 * hidden]`` projection): the two batch levels are walked by stride, nothing
    is copied.  ``tile_variant`` forces a kernel variant (an id that
    ``select_tile`` reports); 0 leaves the choice to the library's per-shape table.
    """
    (A, ao, a_so), (B, bo, b_so), (C, co, c_so), (F, fo, f_so) = (
        _split_levels(A, "A"), _split_levels(B, "B"), _split_levels(C, "C"), _split_levels(F, "F"))
    if not (ao == bo == co == fo):
        raise ValueError("A, B, C, F must agree in their outer batch extent")
    batch, M, K = A.shape
    if B.shape[0] != batch or B.shape[1] != K:
        raise ValueError("B must be [batch, K, L] = [%d, %d, L], got %s" % (batch, K, tuple(B.shape)))
    L = B.shape[2]
    if C.shape[0] != batch or C.shape[1] != L:
        raise ValueError("C must be [batch, L, N] = [%d, %d, N], got %s" % (batch, L, tuple(C.shape)))
    N = C.shape[2]
    if tuple(F.shape) != (batch, M, N):
        raise ValueError("F must be [%d, %d, %d], got %s" % (batch, M, N, tuple(F.shape)))
    if not (A.dtype == B.dtype == C.dtype):
        raise ValueError("A, B, C must share one dtype")
    for t, name in ((A, "A"), (C, "C"), (F, "F")):
        if t.shape[2] > 1 and t.stride(2) != 1:
            raise ValueError("%s rows must be contiguous" % name)
    d = _lib.BmmChainDesc()
    d.abi_version = _lib.ABI_VERSION
    d.in_dtype = _code(A)
    d.acc_dtype = _lib.I32 if A.dtype == torch.int8 else _lib.F64 if A.dtype == torch.float64 else _lib.F32
    d.out_dtype = _code(F)
    d.inter_op = INTER_OPS[inter_op] if isinstance(inter_op, str) else int(inter_op)
    if B.stride(2) == 1 or L == 1:
        d.b_layout = _lib.B_KL
        d.b_row_stride = B.stride(1)
    elif B.stride(1) == 1:
        d.b_layout = _lib.B_LK
        d.b_row_stride = B.stride(2)
    else:
        raise ValueError("B must be contiguous along L or along K")
    d.batch, d.M, d.N, d.K, d.L = batch * ao, M, N, K, L
    d.batch_inner = batch if ao > 1 else 0
    d.a_batch_stride_outer, d.b_batch_stride_outer = a_so, b_so
    d.c_batch_stride_outer, d.f_batch_stride_outer = c_so, f_so
    d.a_batch_stride, d.a_row_stride = A.stride(0), A.stride(1)
    d.b_batch_stride = B.stride(0)
    d.c_batch_stride, d.c_row_stride = C.stride(0), C.stride(1)
    d.f_batch_stride, d.f_row_stride = F.stride(0), F.stride(1)
    d.softmax_scale = float(softmax_scale)
    d.requant_scale = float(requant_scale)
    d.tile_variant = int(tile_variant)
    d.relu_out = int(bool(relu_out))
    return d


def select_tile(desc):
    """Tile the library will use for ``desc`` (validates it as a side effect)."""
    lib = _lib.load()
    tile = _lib.TileParam()
    if isinstance(desc, _lib.BmmChainDesc):
        _lib.check(lib.ditto_bmm_chain_select_tile(ctypes.byref(desc), ctypes.byref(tile)))
    else:
        _lib.check(lib.ditto_conv_chain_select_tile(ctypes.byref(desc), ctypes.byref(tile)))
    return tile


def run_bmm_chain(A, B, C, F, inter_op="cast", softmax_scale=1.0, requant_scale=1.0, aux=None, desc=None,
                  tile_variant=0, relu_out=False):
    """F[b] = epilogue(inter(A[b] . B[b]) . C[b]) as ONE kernel on the current stream.

    ``aux``: for ``inter_op="requant"`` an fp32 tensor of L per-column scales (``None``: use
    ``requant_scale`` for every column)."""
    lib = _lib.load()
    dev = _check_device(A, B, C, F)
    if desc is None:
        desc = bmm_chain_desc(A, B, C, F, inter_op, softmax_scale, requant_scale, tile_variant, relu_out)
    aux_ptr = None
    if aux is not None:
        _check_device(A, aux)
        if aux.dtype != torch.float32 or not aux.is_contiguous() or aux.numel() != desc.L:
            raise ValueError("aux must be a contiguous fp32 tensor of L = %d scales" % desc.L)
        aux_ptr = aux.data_ptr()
    if torch.cuda.current_device() == dev.index:
        # (the common case, kept short: for the smallest chains the host's call path is longer than the kernel)
        rc = lib.ditto_bmm_chain_run(ctypes.byref(desc), A.data_ptr(), B.data_ptr(), C.data_ptr(), aux_ptr,
                                     F.data_ptr(), None, 0, _raw_stream(dev.index))
    else:
        with torch.cuda.device(dev):
            rc = lib.ditto_bmm_chain_run(ctypes.byref(desc), A.data_ptr(), B.data_ptr(), C.data_ptr(), aux_ptr,
                                         F.data_ptr(), None, 0, _raw_stream(dev.index))
    if rc:
        _lib.check(rc)
    return F


def conv_chain_desc(X, W1, W2, Y, pad1=1, stride1=1, pad2=0, stride2=1, inter_op="cast", relu_out=False,
                    groups1=1, tile_variant=0):
    """Fill a ``ditto_conv_chain_desc`` for X[N,C0,H,W], W1[C1,C0/groups1,R1,S1], W2[C2,C1,R2,S2] -> Y.

    ``groups1``: 1 (dense first convolution) or C0 (depthwise, C1 / C0 outputs per input channel).
    ``tile_variant``: 0 (the library's choice) or the kernel to force: a variant id ``select_tile`` reported or a
    family id (3000, 3500, 3600, 3700, 3800, 4000; see ``include/ditto_chain.h``)."""
    for t, name in ((X, "X"), (W1, "W1"), (W2, "W2"), (Y, "Y")):
        if t.dim() != 4 or not t.is_contiguous():
            raise ValueError("%s must be a contiguous 4-D NCHW/KCRS tensor" % name)
    if not (X.dtype == W1.dtype == W2.dtype):
        raise ValueError("X, W1, W2 must share one dtype")
    N, C0, H, W = X.shape
    C1, c0, R1, S1 = W1.shape
    C2, c1, R2, S2 = W2.shape
    if groups1 not in (1, C0):
        raise ValueError("groups1 must be 1 or C0 = %d (depthwise), got %d" % (C0, groups1))
    if c0 * groups1 != C0 or c1 != C1 or C1 % groups1:
        raise ValueError("channel mismatch: X %s, W1 %s, W2 %s" % (tuple(X.shape), tuple(W1.shape), tuple(W2.shape)))
    P1 = (H + 2 * pad1 - R1) // stride1 + 1
    Q1 = (W + 2 * pad1 - S1) // stride1 + 1
    P2 = (P1 + 2 * pad2 - R2) // stride2 + 1
    Q2 = (Q1 + 2 * pad2 - S2) // stride2 + 1
    if tuple(Y.shape) != (N, C2, P2, Q2):
        raise ValueError("Y must be %s, got %s" % ((N, C2, P2, Q2), tuple(Y.shape)))
    d = _lib.ConvChainDesc()
    d.abi_version = _lib.ABI_VERSION
    d.in_dtype = _code(X)
    d.acc_dtype = _lib.F32
    d.out_dtype = _code(Y)
    d.inter_op = INTER_OPS[inter_op] if isinstance(inter_op, str) else int(inter_op)
    d.relu_out = int(bool(relu_out))
    d.N, d.C0, d.H, d.W = N, C0, H, W
    d.C1, d.R1, d.S1, d.pad1, d.stride1 = C1, R1, S1, pad1, stride1
    d.C2, d.R2, d.S2, d.pad2, d.stride2 = C2, R2, S2, pad2, stride2
    d.groups1 = groups1
    d.tile_variant = int(tile_variant)
    return d


_WORKSPACES = {}  # device -> every scratch buffer handed out so far, the current (largest) one last


def _workspace(dev, nbytes):
    """The shared per-device scratch buffer (uint8) of at least ``nbytes`` that ``run_conv_chain`` uses
    when its caller passes none; the library writes the repacked first-convolution weights there on
    every call, so such calls on one device must not overlap.  A buffer that has been handed out is
    never freed: a HIP graph that captured a call keeps a valid pointer when a later, larger request
    makes a new buffer current."""
    bufs = _WORKSPACES.setdefault(dev, [])
    if not bufs or bufs[-1].numel() < nbytes:
        bufs.append(torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=dev))
    return bufs[-1]


def conv_chain_workspace_bytes(desc):
    return _lib.load().ditto_conv_chain_workspace_bytes(ctypes.byref(desc))


def prepare_conv_chain(desc, W1, W2, workspace=None):
    """Repack the weights of a conv chain once (``ditto_conv_chain_prepare``); returns the workspace
    tensor to hand to ``run_conv_chain(..., workspace=ws, prepared=True)`` for as long as W1 / W2 keep
    their values.  ``workspace``: a uint8 tensor of ``conv_chain_workspace_bytes(desc)`` or None to
    allocate one."""
    lib = _lib.load()
    dev = _check_device(W1, W2)
    nbytes = conv_chain_workspace_bytes(desc)
    if workspace is None:
        workspace = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        rc = lib.ditto_conv_chain_prepare(ctypes.byref(desc), W1.data_ptr(), W2.data_ptr(), workspace.data_ptr(),
                                          workspace.numel(), stream)
    _lib.check(rc)
    return workspace


def run_conv_chain(X, W1, W2, Y, pad1=1, stride1=1, pad2=0, stride2=1, inter_op="cast", relu_out=False,
                   desc=None, workspace=None, groups1=1, prepared=False, tile_variant=0):
    """Y = conv2d(inter(conv2d(X, W1)), W2) on the current stream: one fused kernel, preceded by
    a small kernel that repacks W1 into ``workspace`` (a uint8 tensor of
    ``ditto_conv_chain_workspace_bytes``; None: a cached per-device buffer; False: no
    workspace, the fused kernel re-lays W1 out itself, slower).  A depthwise first convolution
    (``groups1 = C0``) is a single kernel and uses no workspace.  ``prepared=True``: ``workspace`` was
    filled by ``prepare_conv_chain`` for these weights; only the fused kernel runs."""
    if prepared and (workspace is None or workspace is False):
        raise ValueError("prepared=True needs the workspace that prepare_conv_chain returned")
    lib = _lib.load()
    dev = _check_device(X, W1, W2, Y)
    if desc is None:
        desc = conv_chain_desc(X, W1, W2, Y, pad1, stride1, pad2, stride2, inter_op, relu_out, groups1, tile_variant)
    ws_bytes = lib.ditto_conv_chain_workspace_bytes(ctypes.byref(desc))
    if workspace is None:
        ws = _workspace(dev, ws_bytes) if ws_bytes else None
    elif workspace is False:
        ws = None
    else:
        ws = workspace
    fn = lib.ditto_conv_chain_run_prepared if prepared else lib.ditto_conv_chain_run
    args = (ctypes.byref(desc), X.data_ptr(), W1.data_ptr(), W2.data_ptr(), Y.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws.numel() * ws.element_size() if ws is not None else 0)
    if torch.cuda.current_device() == dev.index:
        rc = fn(*args, _raw_stream(dev.index))
    else:
        with torch.cuda.device(dev):
            rc = fn(*args, _raw_stream(dev.index))
    if rc:
        _lib.check(rc)
    return Y
