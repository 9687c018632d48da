"""The CPU target of the GEMM chain: the reference's CPU flow (benchmark/chimera/cpu/bmm_bmm_cpu.py:118-276) from
``cpu_intrin`` to ``FusionContext.run`` -> ``build(..., "llvm")`` -> ``f(*inputs, *outputs)``, checked against the
CPU checker (a separate implementation: ``oracle/``) and the fp64 closed form.  No GPU involved."""
import ctypes

import numpy as np
import pytest

import ditto_amd as ditto
from ditto_amd import _cpu_lib, auto_compute as ac, auto_tensorize as at, hardware as hw

F = ac.nn.functional


def _cpu_record(cores=8):
    return hw.hardware_param(num_groups=cores, cacheSizes=[32 * 16, 32 * 1024, 1024 * 1024, 11264 * 1024],
                             bandwidth=[293.72, 81.72, 38.54, 13.14], coresPerCacheLevel=[1.0, 1.0, 1.0, 16.0],
                             tensorWeight=[1.0, 2.0, 1.0, 1.0, 1.0], platform="CPU")


def _flow(ins, outs, dtype="float32", mode="best", tile=(6, 16, 16), with_code=True):
    layer = ac.layer([outs[0].op], inputs=ins)
    sfs = at.build_serial_fusion_state(layer)
    op1, op2 = sfs.first_op, sfs.second_op
    infos = {}
    for op, prefix in ((op1, "gemm1"), (op2, "gemm2")):
        pk, cd = at.cpu_intrin("gemm_noreshape", tile, "avx2", dtype, prefix)
        infos[op] = at.match_info(at.intrinsic_match(op.output(0), pk, ["SameRange"])[0], pk, cd if with_code else "")
    sfs.register_tensorize_axes(list(infos[op1].axis) + list(infos[op2].axis))
    cpu = _cpu_record()
    fc = at.build_fusion_choice(sfs, hw_param=cpu, dtype=dtype, simple_mode=-1)
    state = at.tensorize_hyper_fusion_state(layer, fc, infos)
    ctx = at.build_fusion_context(sfs, layer, state, "", hw_param=cpu, dtype=dtype, searchType="stochastic", mode=mode)
    return layer, sfs, fc, state, ctx


def test_cpu_intrin_generates_the_register_tile_kernel():
    packed, code = at.cpu_intrin(op="gemm_noreshape", shape=(6, 16, 16), isa="avx2", dtype="float32", prefix="gemm1")
    assert packed.compute_intrinsic.name == "gemm1_update" and packed.store_intrinsic is None
    assert str(packed).startswith("PackedIntrinsic(")
    # twelve accumulators, one broadcast per row and step, the two externs of the reference's kernels
    assert code.count("_mm256_fmadd_ps") == 12 and code.count("_mm256_broadcast_ss") == 6
    assert "void gemm1_update(" in code and "void gemm1_reset(" in code
    # the compiled kernel does what it says, on strided tiles
    fn = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p,
                          ctypes.c_long, ctypes.c_long)(_cpu_lib.compile_kernel(code, "gemm1_update"))
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal((6, 40)).astype(np.float32), rng.standard_normal((23, 24)).astype(np.float32)
    c = rng.standard_normal((6, 20)).astype(np.float32)
    want = c.copy()
    want[:, :16] += a[:, :23] @ b[:, :16]
    fn(a.ctypes.data, 40, b.ctypes.data, 24, c.ctypes.data, 20, 23)
    assert np.allclose(c, want, rtol=1e-5, atol=1e-5) and np.array_equal(c[:, 16:], want[:, 16:])
    _, code64 = at.cpu_intrin("gemm", (6, 8, 16), "avx2", "float64", "g")
    assert code64.count("_mm256_fmadd_pd") == 12
    assert at.cpu_intrin("gemm", (6, 64, 64), "avx512", "float32", "g")[1] == ""  # wider than the ymm file: the nest's panels
    assert at.cpu_intrin("exp", (6, 16), "avx2", "float32", "e")[1] == ""
    with pytest.raises(ValueError):
        at.cpu_intrin("gemm", (6, 16, 16), "avx2", "float16")  # the micro-kernels are fp32 / fp64
    with pytest.raises(ValueError):
        at.cpu_intrin("gemm", (6, 16, 16), "sse", "float32")


def test_configuration_1_through_the_cpu_flow(oracle):
    """fp32, batch 1, A[512 x 64] . B[64 x 64] . D[64 x 64], N(0,1) from a seed -- M padded to 516 = 86 x 6 for the
    six-row micro-kernel as the reference's driver does (bmm_bmm_cpu.py:56, 294): every ranked candidate of the
    fusion context, built for the llvm target, against the checker's fused nest and the fp64 closed form at 1e-3."""
    batch, M, N, K, L = 1, 516, 64, 64, 64
    ins, outs = F.BatchGemmGemm(batch, M, N, K, L, "float32", "float32", MI=6, NI=16, KI=16)
    layer, sfs, fc, state, ctx = _flow(ins, outs)
    assert 1 < ctx.size <= 5 and ctx.getComputation(0) == 516 * 64 * 64 * 2
    assert ctx.getFusionLevel(0) == 1  # D_frag's tile under the fused loops: 6 x 64 fp32 = 1.5 KB -> the 32 KB level
    costs = [c.cost for c in ctx.candidates]
    assert costs == sorted(costs) and all(c.m_block % 6 == 0 and c.l_block % 16 == 0 for c in ctx.candidates)
    A, B, C = oracle.make_gemm_chain_inputs(batch, 512, N, K, L, "float32", seed=0)
    A = np.concatenate([A, np.zeros((batch, 4, K), np.float32)], axis=1)  # the padding rows
    want64 = oracle.bmm_chain_f64(A, B, C, inter="cast")
    want_nest = oracle.bmm_chain_fused_f32(A, B, C, inter="cast")
    outs_seen = []
    for i in range(ctx.size):
        sch = ctx.run(i, None)
        assert sch.target == "cpu" and sch.kind == "bmm_chain" and sch.tensorize_param is ctx.candidates[i]
        f = ditto.build(sch, layer.schedule_tensors, "llvm", name="bmm")
        assert f.entry_name == "bmm"
        out = np.full((batch, M, N), np.nan, np.float32)
        f(A, B, C, out)
        assert np.isfinite(out).all()
        assert np.allclose(out, want64, rtol=1e-3, atol=1e-3)
        assert np.linalg.norm(out - want64) / np.linalg.norm(want64) <= 1e-5
        assert np.allclose(out, want_nest, rtol=1e-3, atol=1e-3)
        assert not out[:, 512:].any()  # zero rows in, zero rows out
        outs_seen.append(out)
    # torch CPU tensors and the reference's 5-D packed placeholders (the same memory) are taken too
    import torch

    out_t = torch.full((batch, M, N), float("nan"))
    f(torch.from_numpy(A).view(batch, M // 6, 6, K // 16, 16), torch.from_numpy(B), torch.from_numpy(C), out_t)
    assert np.array_equal(out_t.numpy(), outs_seen[-1])
    cost = f.time_evaluator(f.entry_name, None, min_repeat_ms=0, repeat=3, number=1,
                            f_preproc="cache_flush_cpu_non_first_arg")(A, B, C, out)
    assert 0 < cost.mean < 1.0 and len(cost.results) == 3
    with pytest.raises(IndexError):
        ctx.run(ctx.size, None)


@pytest.mark.parametrize("inter,relu_out", [("relu", False), ("cast", True), ("softmax", False)])
@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_cpu_chain_variants_vs_oracle(oracle, inter, relu_out, dtype):
    """ReLU between / behind the contractions, the softmax chain, fp64 (whose generated tile is 6 x 8): the best, a
    middle and the worst-ranked tiling all give the closed form."""
    batch, M, N, K, L = 3, 96, 32, 48, 80
    rng = np.random.default_rng(7)
    std = 1.0 if inter == "softmax" else 0.5
    A, B, C = (rng.standard_normal(s).astype(dtype) * std for s in ((batch, M, K), (batch, K, L), (batch, L, N)))
    mid = A.astype(np.float64) @ B.astype(np.float64)
    if inter == "softmax":
        ins, outs = F.BatchGemmSoftmaxGemm(batch, M, N, K, L, dtype, dtype, MI=6, NI=16, KI=16, scale=0.25)
        p = np.exp(mid * 0.25 - (mid * 0.25).max(-1, keepdims=True))
        want = (p / p.sum(-1, keepdims=True)) @ C.astype(np.float64)
    else:
        ins, outs = F.BatchGemmGemm(batch, M, N, K, L, dtype, dtype, MI=6, NI=16, KI=16, relu=inter == "relu")
        want = (np.maximum(mid, 0) if inter == "relu" else mid) @ C.astype(np.float64)
    if dtype == "float32":  # ... and the checker agrees with the closed form used here
        assert np.allclose(oracle.bmm_chain_f64(A, B, C, inter=inter, scale=0.25), want, rtol=1e-4, atol=1e-4)
    layer, sfs, fc, state, ctx = _flow(ins, outs, dtype, "survey")
    assert ctx.size >= 6
    tol = 1e-3 if dtype == "float32" else 1e-10
    for i in (0, ctx.size // 2, ctx.size - 1):
        sch = ctx.run(i, None)
        assert sch.inter_op == inter
        sch.relu_out = relu_out
        f = ditto.build(sch, layer.schedule_tensors, "llvm")
        out = np.full(want.shape, np.nan, dtype)
        f(A, B, C, out)
        ref = np.maximum(want, 0) if relu_out else want
        assert np.allclose(out, ref, rtol=tol, atol=tol), (i, np.abs(out - ref).max())


def test_cpu_library_rejects_bad_descriptors_and_ragged_extents_work():
    lib = _cpu_lib.load()
    d = _cpu_lib.CpuChainDesc(abi_version=_cpu_lib.ABI_VERSION, dtype=2, inter_op=0, relu_out=0, batch=2, M=50, N=24, K=40,
                              L=72, a_batch_stride=50 * 40, a_row_stride=40, b_batch_stride=40 * 72, b_row_stride=72,
                              c_batch_stride=72 * 24, c_row_stride=24, f_batch_stride=50 * 24, f_row_stride=24,
                              softmax_scale=1.0, mi=6, ni1=16, ni2=16, m_block=12, l_block=32, threads=3)
    rng = np.random.default_rng(1)
    A, B, C = (rng.standard_normal(s).astype(np.float32) for s in ((2, 50, 40), (2, 40, 72), (2, 72, 24)))
    out = np.full((2, 50, 24), np.nan, np.float32)
    assert lib.ditto_cpu_bmm_chain_run(ctypes.byref(d), A.ctypes.data, B.ctypes.data, C.ctypes.data, out.ctypes.data) == 0
    want = (A.astype(np.float64) @ B) @ C
    assert np.allclose(out, want, rtol=1e-4, atol=1e-3)
    for field, value, word in (("dtype", 0, "fp32 / fp64"), ("m_block", 10, "multiple of mi"), ("mi", 7, "1 .. 6"),
                               ("a_row_stride", 8, "row stride"), ("abi_version", 9, "abi_version")):
        bad = _cpu_lib.CpuChainDesc.from_buffer_copy(d)
        setattr(bad, field, value)
        assert lib.ditto_cpu_bmm_chain_run(ctypes.byref(bad), A.ctypes.data, B.ctypes.data, C.ctypes.data, out.ctypes.data) == -1
        assert word in lib.ditto_cpu_last_error().decode()


def test_targets_are_not_interchangeable():
    ins, outs = F.BatchGemmGemm(1, 96, 32, 32, 64, "float32", "float32", MI=6, NI=16, KI=16)
    layer, sfs, fc, state, ctx = _flow(ins, outs)
    cpu_sch = ctx.run(0, None)
    with pytest.raises(ValueError, match="llvm"):
        ditto.build(cpu_sch, layer.schedule_tensors, "hip")      # a CPU schedule is not silently run on the GPU ...
    hip_sch = at.tensorize_hip(layer, state)
    with pytest.raises(ValueError, match="tensorize_cpu"):
        ditto.build(hip_sch, layer.schedule_tensors, "llvm")     # ... nor a GPU schedule on the CPU
    ins16, outs16 = F.BatchGemmGemm(1, 64, 64, 64, 64, "float16", "float32")
    from tests.test_frontend import _reference_flow

    l16, s16, fc16, st16 = _reference_flow(ins16, outs16, "float16")
    with pytest.raises(ValueError, match="fp32 / fp64"):
        at.tensorize_cpu(l16, st16)
