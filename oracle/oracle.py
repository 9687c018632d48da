"""Python face of the CPU checker (TEST INFRASTRUCTURE, not product code).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
import this module.  It offers

* ctypes wrappers over ``libchain_oracle.so`` (the C restatement in ``chain_oracle.c``;
  build it with ``make -C oracle``), taking and returning numpy arrays, and
* seeded input generators for the five workload configurations, and
* small independent numpy closed forms (``np_*``) that the tests use to pin the C code.

The reference citations for each restated function are in ``chain_oracle.c``.
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libchain_oracle.so")

ROUND_NONE, ROUND_F16, ROUND_BF16, ROUND_F32 = 0, 1, 2, 3
INTER_CAST, INTER_RELU, INTER_SOFTMAX = 0, 1, 2
ROUND_CODES = {"float32": ROUND_F32, "float16": ROUND_F16, "bfloat16": ROUND_BF16, None: ROUND_NONE}
INTER_CODES = {"cast": INTER_CAST, "relu": INTER_RELU, "softmax": INTER_SOFTMAX}

_lib = None


def build():
    """Compile the C restatement (gcc; a few seconds)."""
    subprocess.run(["make", "-C", HERE, "-B", "libchain_oracle.so"], check=True, capture_output=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        fp = ctypes.POINTER(ctypes.c_float)
        i8p = ctypes.POINTER(ctypes.c_int8)
        i32p = ctypes.POINTER(ctypes.c_int32)
        ci = ctypes.c_int
        L.oracle_round_bf16.restype = ctypes.c_float
        L.oracle_round_bf16.argtypes = [ctypes.c_float]
        L.oracle_round_f16.restype = ctypes.c_float
        L.oracle_round_f16.argtypes = [ctypes.c_float]
        L.oracle_round_array.restype = None
        L.oracle_round_array.argtypes = [fp, fp, ctypes.c_longlong, ci]
        L.oracle_bmm_chain_f64.restype = None
        L.oracle_bmm_chain_f64.argtypes = [ci] * 5 + [fp] * 4 + [ci, ctypes.c_double, ci, ci]
        L.oracle_bmm_softmax_ref_emul.restype = None
        L.oracle_bmm_softmax_ref_emul.argtypes = [ci] * 5 + [fp] * 4 + [ci]
        L.oracle_bmm_chain_fused_f32.restype = ci
        L.oracle_bmm_chain_fused_f32.argtypes = [ci] * 5 + [fp] * 4 + [ci, ctypes.c_float, ci, ci, ci, ci, ci]
        L.oracle_requant_shift.restype = ctypes.c_int32
        L.oracle_requant_shift.argtypes = [ctypes.c_int32, ci]
        L.oracle_requant_scale.restype = ctypes.c_int32
        L.oracle_requant_scale.argtypes = [ctypes.c_int32, ctypes.c_float]
        L.oracle_gemm_chain_i8_wrap.restype = None
        L.oracle_gemm_chain_i8_wrap.argtypes = [ci] * 5 + [i8p] * 3 + [ci, i32p, i8p]
        L.oracle_gemm_chain_i8.restype = None
        L.oracle_gemm_chain_i8.argtypes = [ci] * 5 + [i8p] * 3 + [fp, i32p, i8p]
        L.oracle_conv_chain_f32.restype = None
        L.oracle_conv_chain_f32.argtypes = [ci] * 14 + [fp] * 5 + [ci] * 4
        L.oracle_conv_chain_grouped_f32.restype = None
        L.oracle_conv_chain_grouped_f32.argtypes = [ci] * 15 + [fp] * 5 + [ci] * 4
        L.oracle_num_threads.restype = ci
        L.oracle_num_threads.argtypes = []
        _lib = L
    return _lib


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def round_to(x, dtype):
    """Round an fp32 array to the value set of ``dtype`` (kept as fp32), via the C helpers."""
    x = np.asarray(x, dtype=np.float32)
    code = ROUND_CODES[dtype]
    if code == ROUND_NONE:
        return x.copy()
    x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    fp = ctypes.POINTER(ctypes.c_float)
    lib().oracle_round_array(x.ctypes.data_as(fp), out.ctypes.data_as(fp), x.size, code)
    return out


def np_round_to(x, dtype):
    """The same rounding with numpy only (float16 cast; bf16 by integer arithmetic)."""
    x = np.asarray(x, dtype=np.float32)
    if dtype in (None, "float32"):
        return x.copy()
    if dtype == "float16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16).astype(np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) & 0xFFFF0000).astype(np.uint32)
    out = r.view(np.float32).copy()
    nan = np.isnan(x)
    out[nan] = np.nan
    return out


def bmm_chain_f64(A, B, C, inter="cast", scale=1.0, round_mid=None, round_out=None):
    """Closed form in double; A[b,M,K], B[b,K,L], C[b,L,N] -> F[b,M,N] (fp32 array)."""
    A, pa = _f(A)
    B, pb = _f(B)
    C, pc = _f(C)
    batch, M, K = A.shape
    L, N = B.shape[2], C.shape[2]
    assert B.shape == (batch, K, L) and C.shape == (batch, L, N)
    F = np.empty((batch, M, N), dtype=np.float32)
    lib().oracle_bmm_chain_f64(batch, M, N, K, L, pa, pb, pc, F.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                               INTER_CODES[inter], float(scale), ROUND_CODES[round_mid], ROUND_CODES[round_out])
    return F


def bmm_softmax_ref_emul(A, B, C, in_dtype="float16"):
    """The reference's exp / ones-column / divide form with its casts."""
    A, pa = _f(A)
    B, pb = _f(B)
    C, pc = _f(C)
    batch, M, K = A.shape
    L, N = B.shape[2], C.shape[2]
    F = np.empty((batch, M, N), dtype=np.float32)
    lib().oracle_bmm_softmax_ref_emul(batch, M, N, K, L, pa, pb, pc,
                                      F.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), ROUND_CODES[in_dtype])
    return F


def bmm_chain_fused_f32(A, B, C, inter="cast", scale=1.0, round_mid=None, round_out=None, mb=96, lb=256,
                        threads=0, out=None):
    """The fused CPU loop nest (parallel outer blocks, first contraction at the common loop)."""
    A, pa = _f(A)
    B, pb = _f(B)
    C, pc = _f(C)
    batch, M, K = A.shape
    L, N = B.shape[2], C.shape[2]
    F = out if out is not None else np.empty((batch, M, N), dtype=np.float32)
    rc = lib().oracle_bmm_chain_fused_f32(batch, M, N, K, L, pa, pb, pc,
                                          F.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), INTER_CODES[inter],
                                          float(scale), ROUND_CODES[round_mid], ROUND_CODES[round_out], mb, lb,
                                          threads)
    if rc != 0:
        raise MemoryError("oracle_bmm_chain_fused_f32 could not allocate its tiles")
    return F


def gemm_chain_i8(A, B, D, scale, return_mid=False):
    """Exact int8 chain with requantised middle.  A[b,M,K], B[b,K,L], D[b,L,N] int8."""
    A = np.ascontiguousarray(A, dtype=np.int8)
    B = np.ascontiguousarray(B, dtype=np.int8)
    D = np.ascontiguousarray(D, dtype=np.int8)
    if A.ndim == 2:
        A, B, D = A[None], B[None], D[None]
    batch, M, K = A.shape
    L, N = B.shape[2], D.shape[2]
    scale = np.ascontiguousarray(np.broadcast_to(np.asarray(scale, dtype=np.float32), (L,)))
    E = np.empty((batch, M, N), dtype=np.int32)
    mid = np.empty((batch, M, L), dtype=np.int8)
    i8p = ctypes.POINTER(ctypes.c_int8)
    lib().oracle_gemm_chain_i8(batch, M, N, K, L, A.ctypes.data_as(i8p), B.ctypes.data_as(i8p),
                               D.ctypes.data_as(i8p), scale.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                               E.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), mid.ctypes.data_as(i8p))
    return (E, mid) if return_mid else E


def conv_chain_f32(X, W1, W2, pad1=1, stride1=1, pad2=0, stride2=1, relu_mid=False, relu_out=False,
                   round_mid=None, round_out=None, return_mid=False, groups1=1):
    """conv -> (relu) -> round -> conv -> (relu) -> round on NCHW fp32 arrays; ``groups1`` groups the
    first convolution (``groups1 = C0``: depthwise, W1 is [C1, 1, R1, S1])."""
    X, px = _f(X)
    W1, p1 = _f(W1)
    W2, p2 = _f(W2)
    N, C0, H, W = X.shape
    C1, cg, R1, S1 = W1.shape
    C2, _, R2, S2 = W2.shape
    assert C0 % groups1 == 0 and C1 % groups1 == 0 and cg == C0 // groups1
    P1 = (H + 2 * pad1 - R1) // stride1 + 1
    Q1 = (W + 2 * pad1 - S1) // stride1 + 1
    P2 = (P1 + 2 * pad2 - R2) // stride2 + 1
    Q2 = (Q1 + 2 * pad2 - S2) // stride2 + 1
    mid = np.empty((N, C1, P1, Q1), dtype=np.float32)
    Y = np.empty((N, C2, P2, Q2), dtype=np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    lib().oracle_conv_chain_grouped_f32(N, C0, H, W, C1, R1, S1, pad1, stride1, groups1, C2, R2, S2, pad2, stride2,
                                        px, p1, p2, mid.ctypes.data_as(fp), Y.ctypes.data_as(fp), int(relu_mid),
                                        int(relu_out), ROUND_CODES[round_mid], ROUND_CODES[round_out])
    return (Y, mid) if return_mid else Y


def num_threads():
    return lib().oracle_num_threads()


# ---- independent numpy closed forms (used only to pin the C code) ----------------------

def np_bmm_chain(A, B, C, inter="cast", scale=1.0, round_mid=None, round_out=None):
    A, B, C = (np.asarray(x, dtype=np.float64) for x in (A, B, C))
    mid = A @ B
    if inter == "softmax":
        t = mid * scale
        t = t - t.max(axis=-1, keepdims=True)
        e = np.exp(t)
        mid = e / e.sum(axis=-1, keepdims=True)
    else:
        if inter == "relu":
            mid = np.maximum(mid, 0.0)
        if round_mid is not None:
            mid = np_round_to(mid.astype(np.float32), round_mid).astype(np.float64)
    return np_round_to((mid @ C).astype(np.float32), round_out)


def np_requant(mid, scale):
    v = np.rint(mid.astype(np.float32) * np.asarray(scale, dtype=np.float32))
    return np.clip(v, -128, 127).astype(np.int8)


def gemm_chain_i8_wrap(A, B, D, relu=False, return_mid=False):
    """The reference's own int8 chain (bmm_bmm_cuda.py:114-118): the int32 middle result goes back to int8 with
    astype("int8"), i.e. its low byte, optionally behind a ReLU.  A[b,M,K], B[b,K,L], D[b,L,N] int8."""
    A = np.ascontiguousarray(A, dtype=np.int8)
    B = np.ascontiguousarray(B, dtype=np.int8)
    D = np.ascontiguousarray(D, dtype=np.int8)
    if A.ndim == 2:
        A, B, D = A[None], B[None], D[None]
    batch, M, K = A.shape
    L, N = B.shape[2], D.shape[2]
    E = np.empty((batch, M, N), dtype=np.int32)
    mid = np.empty((batch, M, L), dtype=np.int8)
    i8p = ctypes.POINTER(ctypes.c_int8)
    lib().oracle_gemm_chain_i8_wrap(batch, M, N, K, L, A.ctypes.data_as(i8p), B.ctypes.data_as(i8p),
                                    D.ctypes.data_as(i8p), int(bool(relu)), E.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)),
                                    mid.ctypes.data_as(i8p))
    return (E, mid) if return_mid else E


def np_gemm_chain_i8(A, B, D, scale):
    mid = A.astype(np.int64) @ B.astype(np.int64)
    q = np_requant(mid, scale)
    return (q.astype(np.int64) @ D.astype(np.int64)).astype(np.int32)


# ---- seeded inputs of the five workload configurations ---------------------------------

def _normal(rng, shape, std=1.0):
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def make_gemm_chain_inputs(batch, M, N, K, L, dtype="float32", seed=0, std=1.0):
    """A[b,M,K], B[b,K,L], C[b,L,N] iid N(0, std^2), rounded to ``dtype`` (kept as fp32)."""
    rng = np.random.default_rng(seed)
    A = np_round_to(_normal(rng, (batch, M, K), std), dtype)
    B = np_round_to(_normal(rng, (batch, K, L), std), dtype)
    C = np_round_to(_normal(rng, (batch, L, N), std), dtype)
    return A, B, C


def make_attention_inputs(batch, M, L, d, dtype="float16", seed=0):
    """Q[b,M,d], K[b,L,d], V[b,L,d] iid N(0,1) rounded to ``dtype``; the chain's B operand is K^T."""
    rng = np.random.default_rng(seed)
    Q = np_round_to(_normal(rng, (batch, M, d)), dtype)
    K = np_round_to(_normal(rng, (batch, L, d)), dtype)
    V = np_round_to(_normal(rng, (batch, L, d)), dtype)
    return Q, K, V


def make_conv_chain_inputs(N, C0, H, W, C1, C2, R1=3, R2=1, dtype="float16", seed=0, w_std=0.05):
    rng = np.random.default_rng(seed)
    X = np_round_to(_normal(rng, (N, C0, H, W)), dtype)
    W1 = np_round_to(_normal(rng, (C1, C0, R1, R1), w_std), dtype)
    W2 = np_round_to(_normal(rng, (C2, C1, R2, R2), w_std), dtype)
    return X, W1, W2


def make_i8_chain_inputs(M, K, L, N, seed=0):
    """int8 A[M,K], B[K,L], D[L,N] uniform in [-127,127]; scale[L] = 2^-10."""
    rng = np.random.default_rng(seed)
    A = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-127, 128, size=(K, L), dtype=np.int8)
    D = rng.integers(-127, 128, size=(L, N), dtype=np.int8)
    scale = np.full((L,), 2.0 ** -10, dtype=np.float32)
    return A, B, D, scale
