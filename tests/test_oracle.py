"""Pins the CPU checker (oracle/) before anything is compared against it.

The reference holds no golden vectors for the fused-chain path, so each oracle function is
checked against (a) an independent numpy / torch closed form, (b) brute-force Python loops on
tiny shapes, (c) algebraic invariants chosen so that a dropped term, a transposed operand or a
wrong index fails at least one of them.
"""
import itertools

import numpy as np
import pytest
import torch


# ---------------------------------------------------------------------------- roundings
def test_round_f16_matches_numpy_on_all_half_neighbourhoods(oracle):
    # every finite half value, its midpoints to the next value and points just around them
    h = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    nxt = np.arange(1, 0x7C01, dtype=np.uint16).view(np.float16).astype(np.float32)
    nxt[-1] = 65536.0
    mid = ((h.astype(np.float64) + nxt.astype(np.float64)) / 2).astype(np.float32)
    pts = np.concatenate([h, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)),
                          np.array([65519.99, 65520.0, 70000.0, 1e-8, 2.9e-8, 3.0e-8, 0.0], dtype=np.float32)])
    pts = np.concatenate([pts, -pts])
    got = oracle.round_to(pts, "float16")
    want = oracle.np_round_to(pts, "float16")
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_round_bf16_matches_torch(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-20, 20, 20000),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf],
                                 dtype=np.float32)]).astype(np.float32)
    got = oracle.round_to(x, "bfloat16")
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(oracle.np_round_to(x, "bfloat16").view(np.uint32), want.view(np.uint32))
    # ties go to even: 1 + 2^-8 is halfway between 1 and 1 + 2^-7
    assert oracle.round_to(np.float32([1.00390625]), "bfloat16")[0] == 1.0
    assert oracle.round_to(np.float32([1.01171875]), "bfloat16")[0] == np.float32(1.015625)


# ---------------------------------------------------------------------------- GEMM chain
def _brute_chain(A, B, C):
    batch, M, K = A.shape
    L, N = B.shape[2], C.shape[2]
    F = np.zeros((batch, M, N))
    for b, m, n in itertools.product(range(batch), range(M), range(N)):
        acc = 0.0
        for l in range(L):
            d = 0.0
            for k in range(K):
                d += float(A[b, m, k]) * float(B[b, k, l])
            acc += d * float(C[b, l, n])
        F[b, m, n] = acc
    return F


def test_gemm_chain_brute_force_tiny(oracle):
    rng = np.random.default_rng(2)
    A = rng.integers(-3, 4, (2, 5, 3)).astype(np.float32)
    B = rng.integers(-3, 4, (2, 3, 7)).astype(np.float32)
    C = rng.integers(-3, 4, (2, 7, 4)).astype(np.float32)
    want = _brute_chain(A, B, C)  # small integers: exact in every precision
    assert np.array_equal(oracle.bmm_chain_f64(A, B, C), want.astype(np.float32))
    assert np.array_equal(oracle.bmm_chain_fused_f32(A, B, C, mb=6, lb=16), want.astype(np.float32))


@pytest.mark.parametrize("shape", [(1, 512, 64, 64, 64), (3, 100, 24, 40, 72), (2, 13, 17, 5, 33)])
def test_gemm_chain_closed_form(oracle, shape):
    batch, M, N, K, L = shape
    A, B, C = oracle.make_gemm_chain_inputs(batch, M, N, K, L, "float32", seed=3)
    want = oracle.np_bmm_chain(A, B, C)
    got64 = oracle.bmm_chain_f64(A, B, C)
    got32 = oracle.bmm_chain_fused_f32(A, B, C, mb=48, lb=32)
    assert np.allclose(got64, want, rtol=1e-6, atol=1e-6)
    # the reference's own tolerance for this comparison is rtol 1e-3 (test_hyper_fusion_cpu.py:175-177)
    assert np.allclose(got32, want, rtol=1e-4, atol=1e-3)
    # torch as a second library routine
    t = (torch.from_numpy(A).double() @ torch.from_numpy(B).double() @ torch.from_numpy(C).double()).numpy()
    assert np.allclose(got64, t, rtol=1e-6, atol=1e-6)


def test_gemm_chain_invariants(oracle):
    batch, M, N, K, L = 2, 30, 16, 24, 24
    A, B, C = oracle.make_gemm_chain_inputs(batch, M, N, K, L, "float32", seed=4)
    eye = np.broadcast_to(np.eye(K, dtype=np.float32), (batch, K, L)).copy()
    # B = I  =>  F = A.C   (fails if B is applied transposed or an operand is dropped)
    for fn in (oracle.bmm_chain_f64, lambda *a: oracle.bmm_chain_fused_f32(*a, mb=12, lb=16)):
        assert np.allclose(fn(A, eye, C), A @ C, rtol=1e-5, atol=1e-5)
        # linearity in A
        A2 = oracle.make_gemm_chain_inputs(batch, M, N, K, L, "float32", seed=5)[0]
        assert np.allclose(fn(A + 2 * A2, B, C), fn(A, B, C) + 2 * fn(A2, B, C), rtol=1e-4, atol=1e-3)
    # a non-symmetric probe: single one in A, B, C picks one product
    A0 = np.zeros((1, 7, 5), np.float32); B0 = np.zeros((1, 5, 6), np.float32); C0 = np.zeros((1, 6, 4), np.float32)
    A0[0, 2, 3] = 2; B0[0, 3, 1] = 3; C0[0, 1, 2] = 5
    want = np.zeros((1, 7, 4), np.float32); want[0, 2, 2] = 30
    assert np.array_equal(oracle.bmm_chain_f64(A0, B0, C0), want)
    assert np.array_equal(oracle.bmm_chain_fused_f32(A0, B0, C0, mb=6, lb=16), want)


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("inter", ["cast", "relu"])
def test_gemm_chain_mid_rounding(oracle, dtype, inter):
    # the intermediate is cast to in_dtype before the second contraction (bmm_bmm_cuda.py:114-118)
    A, B, C = oracle.make_gemm_chain_inputs(2, 40, 16, 32, 48, dtype, seed=6)
    want = oracle.np_bmm_chain(A, B, C, inter=inter, round_mid=dtype, round_out=dtype)
    got = oracle.bmm_chain_f64(A, B, C, inter=inter, round_mid=dtype, round_out=dtype)
    # identical roundings of values that agree to ~1e-15 relative: allow rare one-ulp flips
    ulp = 2.0 ** -10 if dtype == "float16" else 2.0 ** -7
    assert np.allclose(got, want, rtol=2 * ulp, atol=1e-6)
    assert (got != want).mean() < 0.01
    got32 = oracle.bmm_chain_fused_f32(A, B, C, inter=inter, round_mid=dtype, round_out=dtype, mb=18, lb=32)
    assert np.allclose(got32, want, rtol=4 * ulp, atol=1e-2)
    if inter == "relu":
        assert (oracle.bmm_chain_f64(A, B, np.abs(C), inter="relu") >= 0).all()


# ---------------------------------------------------------------------------- softmax chain
def test_softmax_chain_closed_form_and_torch(oracle):
    Q, K, V = oracle.make_attention_inputs(3, 70, 90, 32, "float32", seed=7)
    B = np.ascontiguousarray(K.transpose(0, 2, 1))
    scale = 1.0 / np.sqrt(32)
    want = oracle.np_bmm_chain(Q, B, V, inter="softmax", scale=scale)
    t = (torch.softmax(torch.from_numpy(Q).double() @ torch.from_numpy(B).double() * scale, -1)
         @ torch.from_numpy(V).double()).numpy()
    assert np.allclose(want, t, rtol=1e-6, atol=1e-7)
    assert np.allclose(oracle.bmm_chain_f64(Q, B, V, inter="softmax", scale=scale), want, rtol=1e-6, atol=1e-7)
    assert np.allclose(oracle.bmm_chain_fused_f32(Q, B, V, inter="softmax", scale=scale, mb=24), want,
                       rtol=1e-4, atol=1e-5)


def test_softmax_chain_invariants(oracle):
    Q, K, V = oracle.make_attention_inputs(2, 20, 48, 16, "float32", seed=8)
    B = np.ascontiguousarray(K.transpose(0, 2, 1))
    for fn in (oracle.bmm_chain_f64, lambda *a, **k: oracle.bmm_chain_fused_f32(*a, mb=12, **k)):
        base = fn(Q, B, V, inter="softmax", scale=0.25)
        # V = ones  =>  O = ones (rows of the softmax sum to one)
        assert np.allclose(fn(Q, B, np.ones_like(V), inter="softmax", scale=0.25), 1.0, atol=1e-6)
        # permuting keys and values together leaves O unchanged
        perm = np.random.default_rng(0).permutation(48)
        assert np.allclose(fn(Q, B[:, :, perm], V[:, perm, :], inter="softmax", scale=0.25), base, atol=1e-5)
        # shifting every score of a row by a constant leaves O unchanged: append a constant
        # column to Q and a matching ones row to B
        Qs = np.concatenate([Q, np.full((2, 20, 1), 7.5, np.float32)], axis=2)
        Bs = np.concatenate([B, np.ones((2, 1, 48), np.float32)], axis=1)
        assert np.allclose(fn(Qs, Bs, V, inter="softmax", scale=0.25), base, atol=1e-5)
        # Q = 0  =>  O = column means of V
        assert np.allclose(fn(np.zeros_like(Q), B, V, inter="softmax", scale=0.25),
                           np.broadcast_to(V.mean(axis=1, keepdims=True), base.shape), atol=1e-6)
        # a huge score selects one value row (and does not overflow thanks to max subtraction)
        Qh = np.zeros_like(Q); Bh = np.zeros_like(B)
        Qh[:, :, 0] = 300.0; Bh[:, 0, 5] = 1.0
        assert np.allclose(fn(Qh, Bh, V, inter="softmax", scale=1.0), np.broadcast_to(V[:, 5:6, :], base.shape),
                           atol=1e-6)


def test_softmax_reference_emulation_matches_closed_form_on_reference_inputs(oracle):
    # the reference checks its exp / ones-column form against torch.softmax on uniform(-1,1)
    # inputs with rtol = atol = 0.1 (bmm_softmax_bmm_wmma_m16n16k16_fp16fp16fp32.py:552-587)
    rng = np.random.default_rng(9)
    batch, M, N, K, L = 2, 32, 16, 16, 64
    Q = oracle.np_round_to(rng.uniform(-1, 1, (batch, M, K)).astype(np.float32), "float16")
    B = oracle.np_round_to(rng.uniform(-1, 1, (batch, K, L)).astype(np.float32), "float16")
    V = oracle.np_round_to(rng.uniform(-1, 1, (batch, L, N)).astype(np.float32), "float16")
    emul = oracle.bmm_softmax_ref_emul(Q, B, V, "float16")
    ideal = oracle.bmm_chain_f64(Q, B, V, inter="softmax", scale=1.0)
    assert np.allclose(emul, ideal, rtol=0.1, atol=0.1)
    assert np.abs(emul - ideal).max() < 5e-3  # the casts cost about three decimal digits
    # fp32 emulation (no casts) agrees much more closely: the ones-column sum IS the softmax sum
    emul32 = oracle.bmm_softmax_ref_emul(Q, B, V, "float32")
    assert np.allclose(emul32, ideal, rtol=1e-3, atol=2e-5)  # +1e-5 in the divisor is the residual
    # and it overflows fp16 as soon as a score exceeds log(65504) = 11.09
    Qb = Q.copy(); Qb[0, 0, :] = 4.0
    Bb = B.copy(); Bb[0, :, 0] = 1.0
    assert not np.isfinite(oracle.bmm_softmax_ref_emul(Qb, Bb, V, "float16")[0, 0]).all()
    assert np.isfinite(oracle.bmm_chain_f64(Qb, Bb, V, inter="softmax")[0, 0]).all()


# ---------------------------------------------------------------------------- int8 chain
def test_requant_integer_and_float_forms_agree(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(10)
    mids = np.concatenate([rng.integers(-(1 << 24) + 1, 1 << 24, 4000), np.arange(-4096, 4097),
                           np.array([512, 1536, -512, -1536, 2560, 130560, 130048, -131584, -130560])])
    for shift in (10, 1, 3, 0):
        s = np.float32(2.0 ** -shift)
        a = np.array([L.oracle_requant_shift(int(m), shift) for m in mids])
        b = np.array([L.oracle_requant_scale(int(m), float(s)) for m in mids])
        c = oracle.np_requant(mids.astype(np.int64), s).astype(np.int64)
        assert np.array_equal(a, b) and np.array_equal(a, c)
    # ties to even, and saturation at both ends
    assert L.oracle_requant_shift(512, 10) == 0 and L.oracle_requant_shift(1536, 10) == 2
    assert L.oracle_requant_shift(-512, 10) == 0 and L.oracle_requant_shift(-1536, 10) == -2
    assert L.oracle_requant_shift(513, 10) == 1 and L.oracle_requant_shift(-513, 10) == -1
    assert L.oracle_requant_shift(200 * 1024, 10) == 127 and L.oracle_requant_shift(-200 * 1024, 10) == -128


def test_i8_chain_exact(oracle):
    A, B, D, scale = oracle.make_i8_chain_inputs(37, 96, 40, 24, seed=11)
    E, mid = oracle.gemm_chain_i8(A, B, D, scale, return_mid=True)
    want = oracle.np_gemm_chain_i8(A, B, D, scale)
    assert E.dtype == np.int32 and np.array_equal(E[0], want)
    assert np.array_equal(mid[0], oracle.np_requant(A.astype(np.int64) @ B.astype(np.int64), scale))
    # brute force on a corner
    m, n = 3, 5
    acc = 0
    for l in range(40):
        d = sum(int(A[m, k]) * int(B[k, l]) for k in range(96))
        q = max(-128, min(127, int(np.rint(np.float32(d) * np.float32(2.0 ** -10)))))
        acc += q * int(D[l, n])
    assert E[0, m, n] == acc
    # per-column scales differ: column l uses scale[l]
    sc = (2.0 ** -np.arange(6, 6 + 40)).astype(np.float32)
    sc[sc < 2.0 ** -12] = 2.0 ** -9
    assert np.array_equal(oracle.gemm_chain_i8(A, B, D, sc)[0], oracle.np_gemm_chain_i8(A, B, D, sc))


def test_i8_wrap_chain_exact(oracle):
    """The reference's own int8 chain (astype("int8") keeps the low byte): against the arithmetic definition of the
    low byte (acc mod 256 taken to [-128, 128)), brute force, numpy's own wrapping cast, and the cases where it
    reduces to the requantised chain (middle results inside int8: scale 1, no saturation, no wrap)."""
    A, B, D, _ = oracle.make_i8_chain_inputs(37, 96, 40, 24, seed=3)
    for relu in (False, True):
        E, mid = oracle.gemm_chain_i8_wrap(A, B, D, relu, return_mid=True)
        acc = A.astype(np.int64) @ B.astype(np.int64)
        if relu:
            acc = np.maximum(acc, 0)
        low = ((acc + 128) % 256) - 128
        assert abs(acc).max() > 127 and np.array_equal(mid[0], low) and (mid[0] != acc).any()
        assert np.array_equal(mid[0], acc.astype(np.int32).astype(np.int8))
        assert E.dtype == np.int32 and np.array_equal(E[0], low @ D.astype(np.int64))
        m, n = 5, 7
        tot = 0
        for l in range(40):
            d = sum(int(A[m, k]) * int(B[k, l]) for k in range(96))
            d = max(d, 0) if relu else d
            d &= 0xff
            tot += (d - 256 if d >= 128 else d) * int(D[l, n])
        assert E[0, m, n] == tot
    # small operands: nothing wraps, and scale 1 requantises to the same bytes
    rng = np.random.default_rng(0)
    As, Bs = rng.integers(-2, 3, (16, 8), dtype=np.int8), rng.integers(-2, 3, (8, 16), dtype=np.int8)
    Ds = rng.integers(-127, 128, (16, 16), dtype=np.int8)
    assert np.array_equal(oracle.gemm_chain_i8_wrap(As, Bs, Ds), oracle.gemm_chain_i8(As, Bs, Ds, 1.0))


# ---------------------------------------------------------------------------- conv chain
def _torch_conv_chain(X, W1, W2, pad1, stride1, pad2, stride2, relu_mid, relu_out):
    x = torch.from_numpy(X).double()
    mid = torch.nn.functional.conv2d(x, torch.from_numpy(W1).double(), padding=pad1, stride=stride1)
    if relu_mid:
        mid = mid.clamp_min(0)
    y = torch.nn.functional.conv2d(mid, torch.from_numpy(W2).double(), padding=pad2, stride=stride2)
    if relu_out:
        y = y.clamp_min(0)
    return y.numpy()


@pytest.mark.parametrize("cfg", [
    # N, C0, H, W, C1, R1, pad1, s1, C2, R2, pad2, s2, relu_mid, relu_out
    (2, 8, 10, 12, 16, 3, 1, 1, 24, 1, 0, 1, False, False),
    (1, 4, 9, 9, 8, 3, 1, 2, 8, 3, 1, 1, True, True),
    (2, 6, 7, 5, 4, 1, 0, 1, 10, 3, 1, 1, True, False),
])
def test_conv_chain_vs_torch(oracle, cfg):
    N, C0, H, W, C1, R1, pad1, s1, C2, R2, pad2, s2, relu_mid, relu_out = cfg
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, R1, R2, "float32", seed=12, w_std=0.3)
    got = oracle.conv_chain_f32(X, W1, W2, pad1, s1, pad2, s2, relu_mid, relu_out)
    want = _torch_conv_chain(X, W1, W2, pad1, s1, pad2, s2, relu_mid, relu_out)
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("cfg", [(2, 8, 9, 11, 1, 1, 12), (1, 4, 10, 10, 16, 2, 8), (1, 6, 7, 9, 2, 1, 5)])
def test_depthwise_conv_chain_vs_torch(oracle, cfg):
    # grouped (depthwise, `factor` outputs per input channel) first convolution against torch conv2d
    N, C0, H, W, factor, s1, C2 = cfg
    rng = np.random.default_rng(21)
    X = rng.standard_normal((N, C0, H, W)).astype(np.float32)
    W1 = (rng.standard_normal((C0 * factor, 1, 3, 3)) * 0.3).astype(np.float32)
    W2 = (rng.standard_normal((C2, C0 * factor, 1, 1)) * 0.3).astype(np.float32)
    got = oracle.conv_chain_f32(X, W1, W2, 1, s1, 0, 1, relu_mid=True, groups1=C0)
    t = torch.nn.functional
    mid = t.conv2d(torch.from_numpy(X).double(), torch.from_numpy(W1).double(), padding=1, stride=s1, groups=C0)
    want = t.conv2d(mid.clamp_min(0), torch.from_numpy(W2).double()).numpy()
    assert np.abs(got - want).max() <= 1e-4
    # one output per input channel and a centre-tap delta filter: the depthwise stage is the identity
    Wd = np.zeros((C0, 1, 3, 3), np.float32)
    Wd[:, 0, 1, 1] = 1.0
    W2i = (rng.standard_normal((C2, C0, 1, 1))).astype(np.float32)
    got = oracle.conv_chain_f32(X, Wd, W2i, 1, 1, 0, 1, groups1=C0)
    assert np.abs(got - np.einsum("kc,nchw->nkhw", W2i[:, :, 0, 0], X)).max() <= 1e-4


def test_conv_chain_delta_kernels(oracle):
    # 3x3 kernel with a single one at (r, s) shifts the image; a 1x1 conv is a channel GEMM
    rng = np.random.default_rng(13)
    X = rng.standard_normal((1, 3, 6, 7)).astype(np.float32)
    W1 = np.zeros((3, 3, 3, 3), np.float32)
    for c in range(3):
        W1[c, c, 0, 2] = 1.0  # y[p][q] = x[p-1][q+1]
    W2 = rng.standard_normal((5, 3, 1, 1)).astype(np.float32)
    got = oracle.conv_chain_f32(X, W1, W2)
    shifted = np.zeros_like(X)
    shifted[:, :, 1:, :-1] = X[:, :, :-1, 1:]
    want = np.einsum("kc,nchw->nkhw", W2[:, :, 0, 0], shifted)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


def test_conv_chain_mid_rounding(oracle):
    X, W1, W2 = oracle.make_conv_chain_inputs(1, 16, 8, 8, 16, 32, dtype="float16", seed=14, w_std=0.1)
    Y, mid = oracle.conv_chain_f32(X, W1, W2, round_mid="float16", round_out="float16", return_mid=True)
    assert np.array_equal(mid, oracle.np_round_to(mid, "float16"))
    assert np.array_equal(Y, oracle.np_round_to(Y, "float16"))
    want = _torch_conv_chain(X, W1, W2, 1, 1, 0, 1, False, False)
    assert np.allclose(Y, want, rtol=5e-3, atol=5e-3)


def test_rounding_floor_of_the_16_bit_types(oracle):
    """What rounding alone costs: the figure the bf16 parity bounds of the GPU tests rest on."""
    x = np.random.default_rng(0).standard_normal(1 << 20).astype(np.float32)
    rel = {dt: float(np.linalg.norm(oracle.np_round_to(x, dt) - x) / np.linalg.norm(x)) for dt in ("bfloat16", "float16")}
    assert 1.6e-3 < rel["bfloat16"] < 1.7e-3 and 2.0e-4 < rel["float16"] < 2.2e-4
    # two independent roundings (probabilities, then output) add in quadrature
    y = oracle.np_round_to(oracle.np_round_to(x, "bfloat16") * np.float32(1.2345), "bfloat16") / np.float32(1.2345)
    assert 2.2e-3 < float(np.linalg.norm(y - x) / np.linalg.norm(x)) < 2.5e-3
