"""Builders of the batched two-GEMM chains.

``BatchGemmSoftmaxGemmMMA`` keeps the reference's signature and op names
(python/ditto/auto_compute/nn/functional/bmm_chain.py:5-105): A_shared, B_shared, D_frag,
exp, C_ext, E_frag, F.  ``BatchGemmGemm`` is the GEMM -> GEMM chain of
benchmark/chimera/cuda/bmm_bmm_cuda.py:69-149 (ops A_shared, B_shared, D_frag, cast, C_ext,
E_frag, F).  They return descriptor DAGs (see ``ditto_amd.te``), not TVM tensors.
"""
import math

from .... import te


def _check_divisible(M, N, K, L, MI, NI, KI):
    assert M % MI == 0, f"M={M}, MI={MI}"
    assert N % NI == 0, f"N={N}, NI={NI}"
    assert K % KI == 0, f"K={K}, KI={KI}"
    assert L % NI == 0, f"L={L}, NI={NI}"
    assert L % KI == 0, f"L={L}, KI={KI}"


def _first_gemm(A, B, batch, M, K, L, MI, NI, KI, in_dtype, acc_dtype):
    A_shared = te.compute(
        [batch, M // MI, K // KI, MI, KI], "A_shared", in_dtype, "pack",
        lambda b, mo, ko, mi, ki: [(A, [b, mo, mi, ko, ki])],
        axis_names=["b", "mo", "ko", "mi", "ki"],
    )
    B_shared = te.compute(
        [batch, K // KI, L // NI, KI, NI], "B_shared", in_dtype, "pack",
        lambda b, ko, lo, ki, li: [(B, [b, ko, ki, lo, li])],
        axis_names=["b", "ko", "lo", "ki", "li"],
    )
    rko = te.reduce_axis([0, K // KI], "rko")
    rki = te.reduce_axis([0, KI], "rki")
    D_frag = te.compute(
        [batch, M // MI, L // NI, MI, NI], "D_frag", acc_dtype, "contract",
        lambda b, mo, lo, mi, li: [(A_shared, [b, mo, rko, mi, rki]), (B_shared, [b, rko, lo, rki, li])],
        axis_names=["b", "mo", "lo", "mi", "li"], reduce_axes=[rko, rki],
    )
    return D_frag


def _second_gemm(P, C, batch, M, L, N, ext_N, MI, NI, KI, in_dtype, acc_dtype, pad_value):
    C_ext = te.compute(
        [batch, L // KI, ext_N // NI, KI, NI], "C_ext", in_dtype, "pad",
        lambda b, lo, no, li, ni: [(C, [b, lo, li, no, ni])],
        axis_names=["b", "lo", "no", "li", "ni"], attrs={"valid_cols": N, "pad_value": pad_value},
    )
    rlo = te.reduce_axis([0, L // KI], "rlo")
    rli = te.reduce_axis([0, KI], "rli")
    E_frag = te.compute(
        [batch, M // MI, ext_N // NI, MI, NI], "E_frag", acc_dtype, "contract",
        lambda b, mo, no, mi, ni: [(P, [b, mo, rlo, mi, rli]), (C_ext, [b, rlo, no, rli, ni])],
        axis_names=["b", "mo", "no", "mi", "ni"], reduce_axes=[rlo, rli],
    )
    return E_frag


def BatchGemmSoftmaxGemmMMA(query, key, value, MI=16, NI=16, KI=16, in_dtype="float16", acc_dtype="float32",
                            scale=1.0):
    """Fused attention chain ``softmax(scale * query . key) . value``.

    query[batch, M, K], key[batch, K, L] (already transposed), value[batch, L, N].
    The reference realises the softmax as ``exp`` on the first accumulator, a column of ones
    appended to ``value`` (so the second GEMM also yields the row sum) and a final divide
    with ``+1e-5``; the descriptor DAG keeps those ops.  ``scale`` (default 1, the
    reference's behaviour) multiplies the scores before the exponential.
    """
    A, B, C = query, key, value
    batch, M, K = A.shape
    _batch, _K, L = B.shape
    _batch2, _L, N = C.shape
    assert _batch == batch and _batch2 == batch and _K == K and _L == L, "operand shapes do not chain"
    _check_divisible(M, N, K, L, MI, NI, KI)
    D_frag = _first_gemm(A, B, batch, M, K, L, MI, NI, KI, in_dtype, acc_dtype)
    exp = te.compute(
        [batch, M // MI, L // NI, MI, NI], "exp", in_dtype, "exp",
        lambda b, mo, lo, mi, li: [(D_frag, [b, mo, lo, mi, li])],
        axis_names=["b", "mo", "lo", "mi", "li"], attrs={"scale": float(scale)},
    )
    ext_N = 2 ** math.ceil(math.log2(N // NI + 1)) * NI
    E_frag = _second_gemm(exp, C, batch, M, L, N, ext_N, MI, NI, KI, in_dtype, acc_dtype, pad_value=1)
    F = te.compute(
        [batch, M, N], "F", in_dtype, "unpack_divide",
        lambda b, m, n: [(E_frag, [b, m, n])],
        axis_names=["b", "m", "n"], attrs={"eps": 1e-5, "denominator_col": ext_N - 1},
    )
    return F


def BatchGemmGemmMMA(A, B, C, MI=16, NI=16, KI=16, in_dtype="float16", acc_dtype="float32", relu=False,
                     requant_scale=None, scale=None, out_dtype=None):
    """GEMM -> GEMM chain on given placeholders: ``F = cast(cast(A.B) . C)`` (optionally
    ReLU on the first accumulator, as test_hyper_fusion_cpu.py:61-67).

    int8 operands with an int32 accumulator (the ("80", "int8", "int32") row of
    bmm_bmm_cuda.py:273-288): the middle result goes back to int8 through a *requantise* op,
    ``saturate(round_to_nearest_even(acc * s))`` with ``s = requant_scale`` for every intermediate
    column or ``scale[l]`` from a float32 placeholder ``scale[L]``, and ``F`` keeps the accumulator
    type unless ``out_dtype`` says otherwise.  Without a scale the chain is the reference's own: the
    middle result and ``F`` go back to int8 with ``astype("int8")`` (:116, :147), which keeps the low
    byte of the int32 accumulator."""
    batch, M, K = A.shape
    _batch, _K, L = B.shape
    _batch2, _L, N = C.shape
    assert _batch == batch and _batch2 == batch and _K == K and _L == L, "operand shapes do not chain"
    _check_divisible(M, N, K, L, MI, NI, KI)
    D_frag = _first_gemm(A, B, batch, M, K, L, MI, NI, KI, in_dtype, acc_dtype)
    requant = requant_scale is not None or scale is not None
    if requant:
        assert not relu, "a requantised middle result has no ReLU variant"
        if scale is not None:
            assert tuple(scale.shape) == (L,), f"scale must be [L]=[{L}], got {scale.shape}"
        mid = te.compute(
            [batch, M // MI, L // NI, MI, NI], "requant", in_dtype, "requant",
            (lambda b, mo, lo, mi, li: [(D_frag, [b, mo, lo, mi, li]), (scale, [lo, li])]) if scale is not None
            else (lambda b, mo, lo, mi, li: [(D_frag, [b, mo, lo, mi, li])]),
            axis_names=["b", "mo", "lo", "mi", "li"],
            attrs={"scale": None if scale is not None else float(requant_scale), "round": "nearest_even",
                   "saturate": True},
        )
        out_dtype = out_dtype or acc_dtype
    else:
        mid = te.compute(
            [batch, M // MI, L // NI, MI, NI], "relu" if relu else "cast", in_dtype, "relu" if relu else "cast",
            lambda b, mo, lo, mi, li: [(D_frag, [b, mo, lo, mi, li])],
            axis_names=["b", "mo", "lo", "mi", "li"],
        )
        out_dtype = out_dtype or in_dtype
    E_frag = _second_gemm(mid, C, batch, M, L, N, N, MI, NI, KI, in_dtype, acc_dtype, pad_value=0)
    F = te.compute(
        [batch, M, N], "F", out_dtype, "unpack_cast",
        lambda b, m, n: [(E_frag, [b, m, n])],
        axis_names=["b", "m", "n"],
    )
    return F


def BatchGemmGemm(batch=12, M=512, N=64, K=64, L=512, in_dtype="float16", acc_dtype="float32", relu=False,
                  MI=16, NI=16, KI=16, requant_scale=None, scale_tensor=False, out_dtype=None):
    """Creates the placeholders too; returns ``([A, B, C], [F])`` like bmm_bmm_cuda.py:69-149.
    int8 / int32: pass ``requant_scale`` (one scale for every intermediate column) or
    ``scale_tensor=True`` (a fourth placeholder ``scale[L]``, float32: returns ``([A, B, C, scale], [F])``)."""
    A = te.placeholder([batch, M, K], name="A", dtype=in_dtype)
    B = te.placeholder([batch, K, L], name="B", dtype=in_dtype)
    C = te.placeholder([batch, L, N], name="C", dtype=in_dtype)
    scale = te.placeholder([L], name="scale", dtype="float32") if scale_tensor else None
    F = BatchGemmGemmMMA(A, B, C, MI, NI, KI, in_dtype, acc_dtype, relu, requant_scale, scale, out_dtype)
    return ([A, B, C, scale] if scale_tensor else [A, B, C]), [F]


def BatchGemmSoftmaxGemm(batch=12, M=512, N=64, K=64, L=512, in_dtype="float16", acc_dtype="float32",
                         scale=1.0, MI=16, NI=16, KI=16):
    """Creates the placeholders too; returns ``([A, B, C], [F])`` like bmm_softmax_bmm_cuda.py:69-155."""
    A = te.placeholder([batch, M, K], name="A", dtype=in_dtype)
    B = te.placeholder([batch, K, L], name="B", dtype=in_dtype)
    C = te.placeholder([batch, L, N], name="C", dtype=in_dtype)
    F = BatchGemmSoftmaxGemmMMA(A, B, C, MI, NI, KI, in_dtype, acc_dtype, scale)
    return [A, B, C], [F]
