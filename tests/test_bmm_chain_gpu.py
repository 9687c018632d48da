"""GPU parity of the fp16 / bf16 fused chains against the CPU checker, through the C ABI.

Tolerances (the workload definition's bar): max-abs-err <= 1e-2 and rel-L2 <= 1e-3 against
the fp32/fp64 closed form on identical seeded inputs.  bf16 carries 8 significant bits, so
rounding the softmax probabilities (as the reference does: ``exp(...).astype(in_dtype)``,
bmm_chain.py:63-70) or the output to bf16 alone costs about 1.6e-3 rel-L2; the bf16 cases
therefore assert 1e-3 where no bf16 rounding of P is on the path (cast chains with fp32
output against the checker that rounds the intermediate the same way) and the measured
quantisation figure + 10 % otherwise, always with max-abs-err <= 1e-2.
"""
import numpy as np
import pytest
import torch

from ditto_amd import chain
from tests.gpu_util import errors, report, to_dev, TORCH_DTYPES

pytestmark = pytest.mark.gpu

MAX_ABS = 1e-2
REL_L2 = 1e-3
# bf16 softmax chains (probabilities and output both rounded to bf16): the largest rel-L2 any case of this
# file reaches is 2.36e-3 (1 x 300 x 128 x 128 x 712; the comment above the long-sequence test derives the
# figure from the rounding floor); bound = that + 10 %.  bf16 cast / relu chains meet the stated 1e-3
# against the checker that rounds where they round (measured: at most 1.1e-4).
REL_L2_BF16_QUANT = 2.6e-3
# the same chains with an fp32 output: only the probabilities are rounded to bf16, which costs 1.66e-3 on
# N(0,1) data (tests/test_oracle.py::test_rounding_floor_of_the_16_bit_types); bound = that floor + 5 %, so a
# kernel error of a few 1e-4 cannot hide under the allowance meant for the rounded output
REL_L2_BF16_P_ONLY = 1.75e-3


def bf16_softmax_bound(out_dtype):
    return REL_L2_BF16_P_ONLY if out_dtype == "float32" else REL_L2_BF16_QUANT


def variants(K, N, b_layout="LK"):
    """0 (the library's own choice) and every kernel variant that can run the head size:
    four waves x 32 rows, four waves x 64 rows, eight waves x 32 rows (staggered phases; software
    pipelined; on the 16x16x32 MFMA with 256-row workgroups and with 384-row ones for the first row blocks), four waves with 64-row workgroups on the 16x16x32 MFMA (head
    size up to 64: a wave owns 16 rows and all keys, or 32 rows and half the keys)."""
    pad = 64 if max(K, N) <= 64 else 128
    return [0] + [pad * 10 + q for q in (1, 2, 8, 9, 6, 7) + ((4, 5) if pad == 64 else ())]


def run_chain(A, B, C, dtype, inter, scale=1.0, b_layout="KL", out_dtype=None, variant=0):
    """A[b,M,K], B[b,K,L], C[b,L,N] fp32 numpy (rounded to dtype) -> F numpy fp32."""
    a, c = to_dev(A, dtype), to_dev(C, dtype)
    if b_layout == "LK":  # keep B^T contiguous and hand over the transposed view
        b = to_dev(np.ascontiguousarray(B.transpose(0, 2, 1)), dtype).transpose(1, 2)
    else:
        b = to_dev(B, dtype)
    f = torch.full((A.shape[0], A.shape[1], C.shape[2]), float("nan"), device=a.device,
                   dtype=TORCH_DTYPES[out_dtype or dtype])
    chain.run_bmm_chain(a, b, c, f, inter, scale, tile_variant=variant)
    torch.cuda.synchronize()
    return f.float().cpu().numpy()


SOFTMAX_SHAPES = [
    # batch, M, N, K, L
    (2, 128, 64, 64, 128),
    (3, 200, 64, 64, 136),    # ragged M and L (tail rows / masked keys)
    (2, 96, 40, 72, 200),     # K != N, both padded inside the kernel
    (1, 16, 16, 16, 16),      # smallest shape the reference builders accept
    (2, 512, 64, 64, 512),    # BERT-base head
    (1, 300, 128, 128, 712),  # 128-wide head
    (12, 208, 64, 64, 208),   # ViT-Base/16 row of the reference's shape table
]


@pytest.mark.parametrize("shape", SOFTMAX_SHAPES)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("b_layout", ["LK", "KL"])
def test_softmax_chain_vs_oracle(oracle, shape, dtype, b_layout):
    batch, M, N, K, L = shape
    scale = 1.0 / np.sqrt(K)
    A, B, C = oracle.make_gemm_chain_inputs(batch, M, N, K, L, dtype, seed=100 + M)
    want = oracle.bmm_chain_f64(A, B, C, inter="softmax", scale=scale)
    for variant in variants(K, N, b_layout):
        for out_dtype in (dtype, "float32"):
            got = run_chain(A, B, C, dtype, "softmax", scale, b_layout, out_dtype, variant)
            assert np.isfinite(got).all(), variant
            mx, rel = errors(got, want)
            if dtype == "bfloat16":
                report("softmax bf16 %s %s variant %d out %s" % (shape, b_layout, variant, out_dtype), mx, rel)
            assert mx <= MAX_ABS, (variant, mx, rel)
            assert rel <= (REL_L2 if dtype == "float16" else bf16_softmax_bound(out_dtype)), (variant, out_dtype, mx, rel)


CAST_SHAPES = [
    (1, 512, 64, 64, 64),     # configuration 1 (shape)
    (2, 128, 64, 64, 128),
    (2, 208, 64, 64, 208),
    (3, 100, 24, 40, 72),     # ragged everything
    (1, 512, 64, 64, 256),    # Mixer-Small row
    (2, 256, 128, 128, 320),
]


@pytest.mark.parametrize("shape", CAST_SHAPES)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("inter", ["cast", "relu"])
def test_cast_chain_vs_oracle(oracle, shape, dtype, inter):
    batch, M, N, K, L = shape
    A, B, C = oracle.make_gemm_chain_inputs(batch, M, N, K, L, dtype, seed=200 + M, std=0.25)
    # the checker rounds the intermediate to in_dtype exactly where the chain does
    want32 = oracle.bmm_chain_f64(A, B, C, inter=inter, round_mid=dtype)
    want = oracle.np_round_to(want32, dtype)
    for b_layout in ("KL", "LK"):
        for variant in variants(K, N, b_layout):
            got32 = run_chain(A, B, C, dtype, inter, 1.0, b_layout, "float32", variant)
            mx, rel = errors(got32, want32)
            # fp32 accumulation order differs; a rounding flip of one intermediate moves the output
            # by about one unit of the intermediate's last place
            assert mx <= MAX_ABS and rel <= REL_L2, (variant, b_layout, mx, rel)
            got = run_chain(A, B, C, dtype, inter, 1.0, b_layout, None, variant)
            mx, rel = errors(got, want)
            if dtype == "bfloat16":
                report("%s bf16 %s %s variant %d" % (inter, shape, b_layout, variant), mx, rel)
            # one bf16 ulp at |x| ~ 4 is 3e-2
            assert mx <= (MAX_ABS if dtype == "float16" else 4e-2), (variant, b_layout, mx, rel)
            assert rel <= REL_L2, (variant, b_layout, mx, rel)
            # and the narrow output is the rounding of the fp32 output (same kernel, cast at the end)
            assert np.array_equal(got, oracle.np_round_to(got32, dtype)), (variant, b_layout)


@pytest.mark.parametrize("shape", [(1, 512, 64, 64, 64), (3, 100, 24, 40, 72), (2, 64, 128, 128, 200)])
@pytest.mark.parametrize("inter", ["cast", "relu", "softmax"])
def test_fp32_chain_vs_oracle(oracle, shape, inter):
    # the reference's fp32, CPU-sized configuration (first shape) and ragged ones, fp32 end to end; softmax: the
    # fp32 BMM -> softmax -> BMM of the reference's CPU benchmark (benchmark/chimera/cpu/bmm_softmax_bmm.py:64-170)
    batch, M, N, K, L = shape
    std = 1.0 if inter == "softmax" else 0.25
    A, B, C = oracle.make_gemm_chain_inputs(batch, M, N, K, L, "float32", seed=300 + M, std=std)
    scale = 0.5 if inter == "softmax" else 1.0
    want = oracle.bmm_chain_f64(A, B, C, inter=inter, scale=scale)
    for b_layout in ("KL", "LK"):
        got = run_chain(A, B, C, "float32", inter, scale, b_layout)
        mx, rel = errors(got, want)
        assert mx <= 1e-4 and rel <= 1e-5, (b_layout, mx, rel)  # fp32 sums of <= 200 terms


@pytest.mark.parametrize("shape", [(1, 512, 64, 64, 64), (3, 100, 24, 40, 72), (2, 64, 128, 128, 200)])
@pytest.mark.parametrize("inter", ["cast", "relu", "softmax"])
def test_fp64_chain_vs_oracle(oracle, shape, inter):
    # the reference's ("80", "float64", "float64") row (benchmark/chimera/cuda/bmm_bmm_cuda.py:273-288): doubles end
    # to end, held to the fp64 closed form at 1e-12
    batch, M, N, K, L = shape
    rng = np.random.default_rng(400 + M)
    std = 1.0 if inter == "softmax" else 0.25
    A, B, C = (rng.standard_normal(sh) * std for sh in ((batch, M, K), (batch, K, L), (batch, L, N)))
    scale = 0.5 if inter == "softmax" else 1.0
    mid = A @ B  # (the checker returns single precision: the closed form in numpy doubles here)
    if inter == "relu":
        mid = np.maximum(mid, 0.0)
    elif inter == "softmax":
        e = np.exp(mid * scale - (mid * scale).max(axis=-1, keepdims=True))
        mid = e / e.sum(axis=-1, keepdims=True)
    want = mid @ C
    assert errors(want, oracle.bmm_chain_f64(A, B, C, inter=inter, scale=scale))[1] <= 1e-6
    a, c = torch.from_numpy(A).cuda(), torch.from_numpy(C).cuda()
    for b_layout in ("KL", "LK"):
        b = torch.from_numpy(np.ascontiguousarray(B.transpose(0, 2, 1))).cuda().transpose(1, 2) if b_layout == "LK" \
            else torch.from_numpy(B).cuda()
        f = torch.full((batch, M, N), float("nan"), device="cuda:0", dtype=torch.float64)
        desc = chain.bmm_chain_desc(a, b, c, f, inter, scale)
        assert chain.select_tile(desc).variant == 1001
        chain.run_bmm_chain(a, b, c, f, inter, scale)
        torch.cuda.synchronize()
        got = f.cpu().numpy()
        assert np.abs(got - want).max() <= 1e-12 * max(1.0, np.abs(want).max()), (b_layout, np.abs(got - want).max())
    with pytest.raises(ValueError):  # mixed types are refused
        chain.run_bmm_chain(a, b, c, torch.empty(batch, M, N, device="cuda:0", dtype=torch.float32), inter, scale)


def test_fused_cpu_nest_agrees_with_gpu(oracle):
    # the CPU baseline (the fused loop nest restatement) and the GPU kernel compute the same chain
    A, B, C = oracle.make_gemm_chain_inputs(1, 512, 64, 64, 64, "float16", seed=7, std=0.25)
    cpu = oracle.bmm_chain_fused_f32(A, B, C, inter="cast", round_mid="float16")
    gpu = run_chain(A, B, C, "float16", "cast", out_dtype="float32")
    mx, rel = errors(gpu, cpu)
    assert mx <= MAX_ABS and rel <= REL_L2


@pytest.mark.parametrize("variant", [641, 642, 648, 649, 646, 644, 645])
def test_softmax_invariants_on_gpu(oracle, variant):
    batch, M, N, K, L = 2, 160, 64, 64, 264
    A, B, C = oracle.make_gemm_chain_inputs(batch, M, N, K, L, "float16", seed=9)
    base = run_chain(A, B, C, "float16", "softmax", 0.125, "LK", "float32", variant)
    # V = ones -> O = ones: the normaliser matches the probabilities that were multiplied
    ones = run_chain(A, B, np.ones_like(C), "float16", "softmax", 0.125, "LK", "float32", variant)
    assert np.abs(ones - 1.0).max() <= 2e-3
    # permuting keys and values together leaves O unchanged (up to accumulation order)
    perm = np.random.default_rng(0).permutation(L)
    got = run_chain(A, np.ascontiguousarray(B[:, :, perm]), np.ascontiguousarray(C[:, perm, :]), "float16",
                    "softmax", 0.125, "LK", "float32", variant)
    assert errors(got, base)[1] <= 5e-4
    # Q = 0 -> O = column means of V
    zero = run_chain(np.zeros_like(A), B, C, "float16", "softmax", 0.125, "KL",
                     "float32", variant)
    assert np.abs(zero - C.mean(axis=1, keepdims=True)).max() <= 1e-3
    # large scores do not overflow (the reference's exp-without-max form does)
    Ah = A.copy()
    Ah[:, :, 0] = 60.0
    hot = run_chain(Ah, B, C, "float16", "softmax", 1.0, "LK", "float32", variant)
    want = oracle.bmm_chain_f64(Ah, B, C, inter="softmax", scale=1.0)
    assert np.isfinite(hot).all() and errors(hot, want)[0] <= MAX_ABS


@pytest.mark.parametrize("variant", [0, 641, 642, 648, 649, 646, 647, 644, 645])
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_running_maximum_paths(oracle, variant, dtype):
    """What the lazily raised row maximum has to survive: every score far below zero from the first key on (the
    maximum starts negative), and keys sorted so that every tile of 64 brings a row maximum far above the last
    (a rescale per tile), with ragged M and L.  (The fp16 kernel that pre-scales A keeps scores relative to the
    maximum; the others subtract it per score; the bf16 kernel on the 16x16x32 MFMA takes no maximum per half
    tile but lowers a row's scale when its sum has grown, and repeats the walk with maxima when a sum overflowed.)"""
    batch, M, N, K, L = 2, 200, 64, 64, 456
    rng = np.random.default_rng(5)
    A = rng.standard_normal((batch, M, K)).astype(np.float32)
    B = rng.standard_normal((batch, K, L)).astype(np.float32)
    C = rng.standard_normal((batch, L, N)).astype(np.float32)
    A[:, :, 0] = 4.0
    cases = {}
    Bn = B.copy()
    Bn[:, 0, :] = -24.0                               # q0 k0 = -96: every score around -96 * scale
    cases["all far below zero"] = Bn
    Br = B.copy()
    Br[:, 0, :] = np.linspace(-20.0, 20.0, L)         # the maximum climbs by about 11 per tile at scale 1
    cases["rising"] = Br
    Bf = B.copy()
    Bf[:, 0, :] = np.linspace(20.0, -20.0, L)         # and the other way: later tiles far below the maximum
    cases["falling"] = Bf
    # a jump of 120 in the exponent from one key to the next, and a short spike of 200 inside the first tile:
    # more than an fp32 (or bf16) probability taken relative to the keys before can hold, so a kernel that
    # watches the row sums instead of taking maxima has to notice and walk the keys again the exact way
    Bs = B.copy()
    Bs[:, 0, :] = -15.0
    Bs[:, 0, 300:] = 15.0
    cases["step up"] = Bs
    Bp = B.copy()
    Bp[:, 0, :] = -25.0
    Bp[:, 0, 40:44] = 25.0
    cases["spike in the first tile"] = Bp
    for name, Bx in cases.items():
        Ar, Bxr, Cr = (oracle.np_round_to(t, dtype) for t in (A, Bx, C))
        got = run_chain(Ar, Bxr, Cr, dtype, "softmax", 1.0, "LK", "float32", variant)
        want = oracle.bmm_chain_f64(Ar, Bxr, Cr, inter="softmax", scale=1.0)
        mx, rel = errors(got, want)
        assert np.isfinite(got).all(), name
        assert mx <= MAX_ABS and rel <= (REL_L2_BF16_P_ONLY if dtype == "bfloat16" else REL_L2), (name, mx, rel)


def test_reference_semantics_on_reference_inputs(oracle):
    # the reference's own check: uniform(-1,1) inputs, scale 1, its exp / ones-column / divide
    # form vs torch softmax at rtol = atol = 0.1 (testing/hyper_fusion/bmm_softmax_bmm_wmma_...py:552-587)
    rng = np.random.default_rng(3)
    batch, M, N, K, L = 12, 512, 64, 64, 512
    A = oracle.np_round_to(rng.uniform(-1, 1, (batch, M, K)).astype(np.float32), "float16")
    B = oracle.np_round_to(rng.uniform(-1, 1, (batch, K, L)).astype(np.float32), "float16")
    C = oracle.np_round_to(rng.uniform(-1, 1, (batch, L, N)).astype(np.float32), "float16")
    emul = oracle.bmm_softmax_ref_emul(A, B, C, "float16")
    got = run_chain(A, B, C, "float16", "softmax", 1.0, "KL")
    assert np.isfinite(got).all()
    # the reference's form breaks where exp or its row sum exceeds the fp16 range (65504): a
    # score above 11.09 gives inf/nan ("nan errors occurs", same file :612-613), a row sum above
    # 65504 an infinite divisor.  Compare on the rows where its form is representable.
    den = np.exp(A.astype(np.float64) @ B.astype(np.float64)).sum(axis=-1)
    ok = np.isfinite(emul).all(axis=-1) & (den < 60000.0)
    assert 0.95 < ok.mean() < 1.0
    assert np.allclose(got[ok], emul[ok], rtol=0.1, atol=0.1)
    assert errors(got[ok], emul[ok])[0] <= 5e-3


def test_attention_full_size_fp16_heads(oracle):
    # the fp16 configuration at its full size: 96 heads of 512 x 64, scale 1/8, every row checked
    batch, M, N, K, L = 96, 512, 64, 64, 512
    A, B, C = oracle.make_gemm_chain_inputs(batch, M, N, K, L, "float16", seed=21)
    want = oracle.bmm_chain_f64(A, B, C, inter="softmax", scale=0.125)
    for variant in variants(K, N):
        got = run_chain(A, B, C, "float16", "softmax", 0.125, "LK", None, variant)
        mx, rel = errors(got, want)
        report("attention fp16 96 x 512 x 64, variant %d" % variant, mx, rel)
        assert mx <= MAX_ABS and rel <= REL_L2, (variant, mx, rel)


# Measured on the long-sequence configuration (64 heads of 4096 x 128, N(0,1) inputs, scale 1/sqrt(128)),
# the same for the three kernel variants to two digits: bf16 rel-L2 2.33e-3 .. 2.35e-3 (max-abs 3.9e-4 ..
# 4.9e-4), fp16 rel-L2 2.87e-4 .. 2.95e-4 (max-abs 4.7e-5 .. 7.0e-5).  The rel-L2 bounds are the largest
# measured figure + 10 %; max-abs, a maximum over a million outputs, gets twice the largest figure.
# The bf16 figure is rounding, not the online softmax: rounding N(0,1) data to bf16 costs rel-L2 1.66e-3 by
# itself (tests/test_oracle.py::test_rounding_floor_of_the_16_bit_types), the chain rounds both the
# probabilities and the output, and 1.66e-3 * sqrt(2) = 2.35e-3.  The fp16 run of the same shape holds the
# online softmax itself, 64 steps and their rescales per row, to the stated 1e-3.
MAX_ABS_BF16_LONG, REL_L2_BF16_LONG = 1.0e-3, 2.6e-3
MAX_ABS_FP16_LONG, REL_L2_FP16_LONG = 1.4e-4, 3.25e-4


@pytest.mark.parametrize("variant", [0, 1282, 1288, 1289, 1286, 1287])
def test_attention_full_size_fp16_long_sequence(oracle, variant):
    # the long-sequence shape in fp16, where the stated bar (1e-2 / 1e-3) is reachable: 64 online-softmax
    # steps per row, every variant; three whole heads and a row block of every head against the closed form
    batch, S, d = 64, 4096, 128
    scale = d ** -0.5
    dev = "cuda:0"
    g = torch.Generator(device="cpu").manual_seed(34)
    q = torch.randn(batch, S, d, generator=g).to(torch.float16)
    k = torch.randn(batch, S, d, generator=g).to(torch.float16)
    v = torch.randn(batch, S, d, generator=g).to(torch.float16)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    out = torch.full((batch, S, d), float("nan"), device=dev, dtype=torch.float16)
    chain.run_bmm_chain(qd, kd.transpose(1, 2), vd, out, "softmax", scale, tile_variant=variant)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    assert np.isfinite(got).all()
    qn, kn, vn = q.float().numpy(), k.float().numpy(), v.float().numpy()
    for h in (0, 17, 63):
        want = oracle.bmm_chain_f64(qn[h:h + 1], np.ascontiguousarray(kn[h:h + 1].transpose(0, 2, 1)), vn[h:h + 1],
                                    inter="softmax", scale=scale)
        mx, rel = errors(got[h:h + 1], want)
        report("attention fp16 64 x 4096 x 128, variant %d, head %d" % (variant, h), mx, rel)
        assert mx <= MAX_ABS and rel <= REL_L2, (h, mx, rel)                      # the stated bar
        assert mx <= MAX_ABS_FP16_LONG and rel <= REL_L2_FP16_LONG, (h, mx, rel)  # measured + 10 %
    rows = slice(3000, 3032)
    want = oracle.bmm_chain_f64(np.ascontiguousarray(qn[:, rows]), np.ascontiguousarray(kn.transpose(0, 2, 1)), vn,
                                inter="softmax", scale=scale)
    mx, rel = errors(got[:, rows], want)
    report("attention fp16 64 x 4096 x 128, variant %d, rows 3000-3031 of every head" % variant, mx, rel)
    assert mx <= MAX_ABS_FP16_LONG and rel <= REL_L2_FP16_LONG, (mx, rel)
    # scores shifted far from zero: keys scaled up make row maxima of +-40 and more in the exponent, so
    # the running maximum is raised many times along a row
    big = (kd.float() * 6.0).to(torch.float16)
    chain.run_bmm_chain(qd[:2], big[:2].transpose(1, 2), vd[:2], out[:2], "softmax", scale, tile_variant=variant)
    torch.cuda.synchronize()
    want = oracle.bmm_chain_f64(qn[:2, :256], np.ascontiguousarray(big[:2].float().cpu().numpy().transpose(0, 2, 1)),
                                vn[:2], inter="softmax", scale=scale)
    mx, rel = errors(out[:2, :256].float().cpu().numpy(), want)
    report("attention fp16 2 x 4096 x 128 with keys x 6, variant %d" % variant, mx, rel)
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)


@pytest.mark.parametrize("variant", [0, 1282, 1288, 1289, 1286, 1287])
def test_attention_full_size_bf16_long_sequence(oracle, variant):
    # the bf16 configuration at its full size (64 heads of 4096 x 128).  The CPU closed form over
    # all of it would take minutes, so: every row of three heads chosen across the batch, one
    # row block of every head, and size-independent properties over the whole output.
    batch, S, d = 64, 4096, 128
    scale = d ** -0.5
    dev = "cuda:0"
    g = torch.Generator(device="cpu").manual_seed(33)
    q = torch.randn(batch, S, d, generator=g).to(torch.bfloat16)
    k = torch.randn(batch, S, d, generator=g).to(torch.bfloat16)
    v = torch.randn(batch, S, d, generator=g).to(torch.bfloat16)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    out = torch.full((batch, S, d), float("nan"), device=dev, dtype=torch.bfloat16)
    chain.run_bmm_chain(qd, kd.transpose(1, 2), vd, out, "softmax", scale, tile_variant=variant)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    assert np.isfinite(got).all()
    qn, kn, vn = q.float().numpy(), k.float().numpy(), v.float().numpy()
    for h in (0, 31, 63):  # whole heads
        want = oracle.bmm_chain_f64(qn[h:h + 1], np.ascontiguousarray(kn[h:h + 1].transpose(0, 2, 1)), vn[h:h + 1],
                                    inter="softmax", scale=scale)
        mx, rel = errors(got[h:h + 1], want)
        report("attention bf16 64 x 4096 x 128, variant %d, head %d" % (variant, h), mx, rel)
        assert mx <= MAX_ABS_BF16_LONG and rel <= REL_L2_BF16_LONG, (h, mx, rel)
    rows = slice(1000, 1032)  # one row block of every head (straddles no tile boundary specially)
    want = oracle.bmm_chain_f64(np.ascontiguousarray(qn[:, rows]), np.ascontiguousarray(kn.transpose(0, 2, 1)), vn,
                                inter="softmax", scale=scale)
    mx, rel = errors(got[:, rows], want)
    report("attention bf16 64 x 4096 x 128, variant %d, rows 1000-1031 of every head" % variant, mx, rel)
    assert mx <= MAX_ABS_BF16_LONG and rel <= REL_L2_BF16_LONG, (mx, rel)
    # values all ones -> output all ones (the normaliser is the sum of what was multiplied)
    ones = torch.ones_like(vd)
    chain.run_bmm_chain(qd, kd.transpose(1, 2), ones, out, "softmax", scale, tile_variant=variant)
    torch.cuda.synchronize()
    assert (out.float() - 1.0).abs().max().item() <= 8e-3  # one bf16 ulp below 1 is 3.9e-3
    # convexity: every output lies within the column range of V of its head
    chain.run_bmm_chain(qd, kd.transpose(1, 2), vd, out, "softmax", scale, tile_variant=variant)
    torch.cuda.synchronize()
    lo = vd.float().amin(dim=1, keepdim=True)
    hi = vd.float().amax(dim=1, keepdim=True)
    o32 = out.float()
    assert bool(((o32 >= lo - 1e-2) & (o32 <= hi + 1e-2)).all())
    # rows of Q permuted -> rows of the output permuted the same way.  Not bit for bit: the
    # running maximum is raised for all rows of a wave at once, so a row's rescale history (and
    # with it the last bit before rounding) depends on its neighbours; a few outputs move by
    # one bf16 unit in the last place.
    perm = torch.randperm(S, generator=g).to(dev)
    out2 = torch.empty_like(out)
    chain.run_bmm_chain(qd[:, perm].contiguous(), kd.transpose(1, 2), vd, out2, "softmax", scale, tile_variant=variant)
    torch.cuda.synchronize()
    a, b = out2.float(), out[:, perm].float()
    assert float((a != b).float().mean()) <= 1e-2
    assert float((a - b).norm() / b.norm()) <= 5e-4
    assert bool(((a - b).abs() <= 2.0 ** -7 * b.abs() + 1e-6).all())


@pytest.mark.parametrize("variant", [0, 1281, 1288, 1289])
def test_gemm_chain_full_size_bf16(oracle, variant):
    # the large GEMM-chain point of the benchmark, (A.B).D with the cast between, 64 x (4096 x 128 x
    # 4096 x 128) bf16, B as [K][L] like the reference's operand.  The checker over all of it would take
    # minutes: whole entries across the batch, one row block of every entry, and properties.
    batch, M, K, L, N = 64, 4096, 128, 4096, 128
    dev = "cuda:0"
    g = torch.Generator(device="cpu").manual_seed(35)
    a = (torch.randn(batch, M, K, generator=g) * 0.25).to(torch.bfloat16)
    b = (torch.randn(batch, K, L, generator=g) * 0.25).to(torch.bfloat16)
    c = (torch.randn(batch, L, N, generator=g) / 64).to(torch.bfloat16)  # keeps the outputs O(1)
    ad, bd, cd = a.to(dev), b.to(dev), c.to(dev)
    out = torch.full((batch, M, N), float("nan"), device=dev, dtype=torch.bfloat16)
    chain.run_bmm_chain(ad, bd, cd, out, "cast", 1.0, tile_variant=variant)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    assert np.isfinite(got).all()
    an, bn, cn = a.float().numpy(), b.float().numpy(), c.float().numpy()
    for h in (0, 40, 63):
        want = oracle.bmm_chain_f64(an[h:h + 1], bn[h:h + 1], cn[h:h + 1], inter="cast", round_mid="bfloat16")
        mx, rel = errors(got[h:h + 1], oracle.np_round_to(want.astype(np.float32), "bfloat16"))
        report("GEMM chain bf16 64 x 4096 x 128, variant %d, head %d" % (variant, h), mx, rel)
        assert rel <= REL_L2 and mx <= 4e-2, (h, mx, rel)  # one bf16 ulp at |x| ~ 4 is 3e-2
    rows = slice(3000, 3040)
    want = oracle.bmm_chain_f64(np.ascontiguousarray(an[:, rows]), bn, cn, inter="cast", round_mid="bfloat16")
    mx, rel = errors(got[:, rows], oracle.np_round_to(want.astype(np.float32), "bfloat16"))
    assert rel <= REL_L2 and mx <= 4e-2, (mx, rel)
    # B = [I | 0]: the middle result is A itself (exact in bf16), so F = A . C[:K] -- one GEMM
    eye = torch.zeros(batch, K, L, dtype=torch.bfloat16, device=dev)
    eye[:, torch.arange(K), torch.arange(K)] = 1
    chain.run_bmm_chain(ad, eye, cd, out, "cast", 1.0, tile_variant=variant)
    torch.cuda.synchronize()
    want_d = torch.bmm(ad.float(), cd[:, :K].float())
    # (against an unrounded fp32 product: the bf16 rounding of the output alone is 1.66e-3)
    assert float((out.float() - want_d).norm() / want_d.norm()) <= REL_L2_BF16_QUANT
    # rows of A permuted -> rows of F permuted, bit for bit (no cross-row state in this chain)
    perm = torch.randperm(M, generator=g).to(dev)
    chain.run_bmm_chain(ad, bd, cd, out, "cast", 1.0, tile_variant=variant)
    out2 = torch.empty_like(out)
    chain.run_bmm_chain(ad[:, perm].contiguous(), bd, cd, out2, "cast", 1.0, tile_variant=variant)
    torch.cuda.synchronize()
    assert torch.equal(out2, out[:, perm])


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("cfg", [(2, 3, 200, 64), (1, 16, 256, 128), (8, 12, 512, 64)])
def test_multi_head_attention_module(oracle, dtype, cfg):
    # packed [batch, M, 3*hidden] projection in, [batch, M, hidden] out, heads walked by stride;
    # checked against the reference's own formulation (split, reshape, transpose, chain, merge:
    # nn/module/self_attention.py:46-73) evaluated in fp64 on the CPU
    from ditto_amd import auto_compute as ac

    batch, heads, M, d = cfg
    hidden = heads * d
    rng = np.random.default_rng(heads + M)
    qkv = oracle.np_round_to(rng.standard_normal((batch, M, 3 * hidden)).astype(np.float32), dtype)
    mha = ac.nn.module.MultiHeadAttentionMMA(heads, hidden, in_dtype=dtype, scale=None)
    x = to_dev(qkv, dtype)
    out = mha(x)
    torch.cuda.synchronize()
    assert out.shape == (batch, M, hidden) and out.is_contiguous()
    q, k, v = (qkv[:, :, i * hidden:(i + 1) * hidden].reshape(batch, M, heads, d).transpose(0, 2, 1, 3)
               .reshape(batch * heads, M, d) for i in range(3))
    want = oracle.bmm_chain_f64(q, np.ascontiguousarray(k.transpose(0, 2, 1)), v, inter="softmax", scale=d ** -0.5)
    want = want.reshape(batch, heads, M, d).transpose(0, 2, 1, 3).reshape(batch, M, hidden)
    mx, rel = errors(out.float().cpu().numpy(), want)
    if dtype == "bfloat16":
        report("multi-head attention bf16 %s" % (cfg,), mx, rel)
    assert mx <= MAX_ABS and rel <= (REL_L2 if dtype == "float16" else REL_L2_BF16_QUANT), (mx, rel)
    # same numbers as the chain on materialised per-head tensors (bit for bit: same kernel, same order)
    qd, kd, vd = (to_dev(np.ascontiguousarray(t), dtype) for t in (q, k, v))
    ref = torch.empty(batch * heads, M, d, device=x.device, dtype=x.dtype)
    chain.run_bmm_chain(qd, kd.transpose(1, 2), vd, ref, "softmax", d ** -0.5,
                        tile_variant=chain.select_tile(chain.bmm_chain_desc(*mha.head_views(x), out.view(batch, M, heads, d).permute(0, 2, 1, 3), "softmax", d ** -0.5)).variant)
    torch.cuda.synchronize()
    assert torch.equal(ref.view(batch, heads, M, d).permute(0, 2, 1, 3).reshape(batch, M, hidden), out)


def test_tile_variant_tuning_round_trip(tmp_path, oracle):
    # measure the variants for one shape, log them in the reference's format, reuse the log
    from ditto_amd.auto_schedule.schedulers import chimera_integrate as ci

    dev = "cuda:0"
    torch.manual_seed(1)
    q, k, v = (torch.randn(16, 1024, 64, device=dev).half() for _ in range(3))
    f = torch.empty_like(q)
    log = str(tmp_path / "chimera_tune.log")
    key = ci.workload_key(chain.bmm_chain_desc(q, k.transpose(1, 2), v, f, "softmax", 0.125))
    best = ci.select_tile_variant(key, log, q, k.transpose(1, 2), v, f, "softmax", 0.125, top=3, min_repeat_ms=5)
    records = ci.load_best_records(log)
    assert len(open(log).read().strip().splitlines()) == 3
    assert records[key]["record"]["variant"] == best.record["variant"] and 0 < best.value < 5.0
    assert ci.auto_schedule_bmm_chain_hip(key, log, q, k.transpose(1, 2), v, f, "softmax", 0.125) == best.record["variant"]
    chain.run_bmm_chain(q, k.transpose(1, 2), v, f, "softmax", 0.125, tile_variant=best.record["variant"])
    ref = torch.softmax(q.float() @ k.float().transpose(1, 2) * 0.125, -1) @ v.float()
    assert (f.float() - ref).abs().max().item() <= MAX_ABS


def test_strided_views_and_errors():
    dev = "cuda:0"
    torch.manual_seed(0)
    # operands that are slices of larger buffers (row stride > row extent)
    big_a = torch.randn(2, 128, 96, device=dev).half()
    big_b = torch.randn(2, 160, 96, device=dev).half()
    big_c = torch.randn(2, 160, 96, device=dev).half()
    a, bt, c = big_a[:, :, :64], big_b[:, :, 16:80], big_c[:, :, 8:72]
    f = torch.empty(2, 128, 64, device=dev, dtype=torch.float16)
    chain.run_bmm_chain(a, bt.transpose(1, 2), c, f, "softmax", 0.125)
    ref = torch.softmax(a.float() @ bt.float().transpose(1, 2) * 0.125, -1) @ c.float()
    assert (f.float() - ref).abs().max().item() <= MAX_ABS
    # the output as a slice too.  Rows that all start on 16 bytes (row stride 96) leave through LDS as whole rows,
    # others (row stride 100) are stored from registers, four columns per lane: every variant gives the same bits
    for variant in variants(64, 64, "LK"):
        chain.run_bmm_chain(a, bt.transpose(1, 2), c, f, "softmax", 0.125, tile_variant=variant)
        for width in (96, 100):
            big_f = torch.full((2, 128, width), float("nan"), device=dev, dtype=torch.float16)
            chain.run_bmm_chain(a, bt.transpose(1, 2), c, big_f[:, :, 8:72], "softmax", 0.125, tile_variant=variant)
            assert torch.equal(big_f[:, :, 8:72], f), (variant, width)
            assert torch.isnan(big_f[:, :, :8]).all() and torch.isnan(big_f[:, :, 72:]).all(), (variant, width)
    with pytest.raises(ValueError):
        chain.run_bmm_chain(a[:, :, :60], bt[:, :, :60].transpose(1, 2), c, f, "softmax", 0.125)
    with pytest.raises(ValueError):
        chain.run_bmm_chain(a, bt.transpose(1, 2), c, f[:, :64], "softmax", 0.125)
    with pytest.raises(NotImplementedError):
        wide = torch.randn(2, 128, 256, device=dev).half()
        chain.run_bmm_chain(wide, torch.randn(2, 256, 64, device=dev).half(),
                            torch.randn(2, 64, 64, device=dev).half(), f, "cast")
    with pytest.raises(ValueError):
        chain.run_bmm_chain(a.cpu(), bt.transpose(1, 2).cpu(), c.cpu(), f.cpu(), "softmax", 0.125)


def test_fp16_accumulator_request_is_served_in_fp32():
    """The reference's ("80", "float16", "float16") rows (benchmark/chimera/cuda/bmm_bmm_cuda.py:273-288): an fp16
    accumulator asked for with fp16 operands runs the same kernels on the MFMA's fp32 accumulator -- the same bits as
    the fp32 request; a bf16 accumulator is no row of the reference and stays refused."""
    from ditto_amd import _lib
    dev = "cuda:0"
    torch.manual_seed(1)
    a, bt, c = (torch.randn(2, 128, 64, device=dev).half() for _ in range(3))
    f32, f16 = (torch.empty(2, 128, 64, device=dev, dtype=torch.float16) for _ in range(2))
    for inter in ("softmax", "cast"):
        chain.run_bmm_chain(a, bt.transpose(1, 2), c, f32, inter, 0.125)
        desc = chain.bmm_chain_desc(a, bt.transpose(1, 2), c, f16, inter, 0.125)
        desc.acc_dtype = _lib.F16
        chain.run_bmm_chain(a, bt.transpose(1, 2), c, f16, inter, 0.125, desc=desc)
        assert torch.equal(f16, f32)
    ab, bb, cb = a.bfloat16(), bt.bfloat16(), c.bfloat16()
    fb = torch.empty(2, 128, 64, device=dev, dtype=torch.bfloat16)
    desc = chain.bmm_chain_desc(ab, bb.transpose(1, 2), cb, fb, "cast")
    desc.acc_dtype = _lib.BF16
    with pytest.raises(NotImplementedError):
        chain.run_bmm_chain(ab, bb.transpose(1, 2), cb, fb, "cast", desc=desc)


def test_front_end_end_to_end(oracle):
    import ditto_amd as ditto
    from ditto_amd import auto_compute as ac, auto_tensorize as at, hardware as hw

    batch, M, N, K, L = 8, 256, 64, 64, 256
    ins, outs = ac.nn.functional.BatchGemmSoftmaxGemm(batch, M, N, K, L, "float16", "float32", scale=0.125)
    A, B, C = ins
    (F,) = outs
    E_frag = F.op.input_tensors[0]
    exp, C_ext = E_frag.op.input_tensors
    D_frag = exp.op.input_tensors[0]
    b, m, n, mi, ni = E_frag.op.axis
    rlo, rli = E_frag.op.reduce_axis
    fuse_choice = at.fusion_choice(D_frag.op, E_frag.op, [b, m, n, rlo, mi, ni, rli], 3)
    p1 = at.cuda_wmma(16, 16, 16, "float16", "float32", "shared")
    p2 = at.cuda_wmma(16, 16, 16, "float16", "float32", "global")
    layer = ac.layer([F.op], inputs=[A, B, C])
    state = at.tensorize_hyper_fusion_state(layer, fuse_choice, {
        D_frag.op: at.match_info(at.intrinsic_match(D_frag, p1, ["InnerMost", "SameRange"])[0], p1),
        E_frag.op: at.match_info(at.intrinsic_match(E_frag, p2, ["InnerMost", "SameRange"])[0], p2)})
    sch = at.tensorize_cuda(layer, state, hw.query_hw_param("gpu.hip.MI355X"), at.cuda_tensorize_param())
    func = ditto.build(sch, layer.schedule_tensors, "hip")
    a_np, b_np, c_np = oracle.make_gemm_chain_inputs(batch, M, N, K, L, "float16", seed=5)
    args = [to_dev(a_np, "float16"), to_dev(b_np, "float16"), to_dev(c_np, "float16"),
            torch.empty(batch, M, N, device="cuda:0", dtype=torch.float16)]
    func(*args)
    torch.cuda.synchronize()
    want = oracle.bmm_chain_f64(a_np, b_np, c_np, inter="softmax", scale=0.125)
    mx, rel = errors(args[3].float().cpu().numpy(), want)
    assert mx <= MAX_ABS and rel <= REL_L2
    t = func.time_evaluator(func.entry_name, None, min_repeat_ms=20)(*args)
    assert 0 < t.mean < 1e-2
    with pytest.raises(ValueError):
        func(*args[:3])


def test_reference_test_flow_with_build_fusion_choice(oracle):
    """python_test/auto_tensorize/test_hyper_fusion.py:833-910 (test_tensorize_cuda_run) against this package:
    serial fusion state -> intrinsic match -> register_tensorize_axes -> build_fusion_choice ->
    tensorize_hyper_fusion_state -> tensorize_cuda -> build -> time_evaluator, on the reference's own
    uniform(-1, 1) inputs; the result is checked, which the reference's test does not do."""
    import ditto_amd as ditto
    from ditto_amd import auto_compute as ac, auto_tensorize as at, hardware as hw

    ins, outs = ac.nn.functional.BatchGemmSoftmaxGemm()  # the reference's defaults: 12 x 512 x 64 x 64 x 512
    layer = ac.layer([outs[0].op], inputs=ins)
    sfs = at.build_serial_fusion_state(layer)
    op1, op2 = sfs.first_op, sfs.second_op

    def get_match_info(op, store_scope):
        packed = at.cuda_wmma(16, 16, 16, "float16", "float32", store_scope)
        choice = at.intrinsic_match(op.output(0), packed, ["InnerMost", "SameRange"])[0]
        return at.match_info(choice, packed, impl="")

    first_match_info = get_match_info(op1, "shared")
    second_match_info = get_match_info(op2, "global")
    sfs.register_tensorize_axes(list(first_match_info.axis) + list(second_match_info.axis))
    V100 = hw.query_hw_param("gpu.cuda.V100")
    fuse_choice = at.build_fusion_choice(sfs, hw_param=V100, dtype="float32", simple_mode=-1)
    tensorize_state = at.tensorize_hyper_fusion_state(layer, fuse_choice, {op1: first_match_info, op2: second_match_info})
    tensorize_param = at.cuda_tensorize_param(warp_size=32, ty_size=4, tz_size=2, input_vector_len=4, serial_y=2,
                                              serial_z=1, block_rx=8, warp_rx=4, block_ry=1, warp_ry=4,
                                              unroll_steps=512)
    sch = at.tensorize_cuda(layer, tensorize_state, V100, tensorize_param)
    func = ditto.build(sch, layer.schedule_tensors, "hip")
    rng = np.random.default_rng(0)
    inputs_np = [oracle.np_round_to(rng.uniform(-1, 1, [int(x) for x in y.shape]).astype(np.float32), "float16")
                 for y in ins]
    inputs = [to_dev(x, "float16") for x in inputs_np]
    outputs = [torch.full(tuple(y.shape), float("nan"), device="cuda:0", dtype=torch.float16) for y in outs]
    evaluator = func.time_evaluator(func.entry_name, None, min_repeat_ms=50)
    cost = evaluator(*inputs, *outputs).mean * 1e3
    assert 0 < cost < 1.0  # ms
    want = oracle.bmm_chain_f64(*inputs_np, inter="softmax", scale=1.0)
    mx, rel = errors(outputs[0].float().cpu().numpy(), want)
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)
    # the descriptor is filled once and reused; a forced variant travels from the schedule to the call
    assert len(func._descs) == 1
    sch8 = at.tensorize_hip(layer, tensorize_state, tile_variant=648)
    f8 = ditto.build(sch8, layer.schedule_tensors, "hip")
    f8(*inputs, *outputs)
    torch.cuda.synchronize()
    assert next(iter(f8._descs.values())).tile_variant == 648
    assert errors(outputs[0].float().cpu().numpy(), want)[1] <= REL_L2


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32"])
def test_relu_after_the_second_contraction(oracle, dtype):
    # relu_out: the slot a fused activation layer lands in (chimera.graph_fusion)
    batch, M, N, K, L = 2, 200, 64, 40, 136
    A, B, C = oracle.make_gemm_chain_inputs(batch, M, N, K, L, dtype if dtype != "float32" else "float16", seed=9, std=0.25)
    want = np.maximum(oracle.bmm_chain_f64(A, B, C, inter="relu", round_mid=None if dtype == "float32" else dtype), 0.0)
    dev = "cuda:0"
    if dtype == "float32":
        a, b, c = (torch.from_numpy(x).to(dev) for x in (A, B, C))
    else:
        a, b, c = to_dev(A, dtype), to_dev(B, dtype), to_dev(C, dtype)
    for variant in ([0] if dtype == "float32" else variants(K, N, "KL")):
        f = torch.full((batch, M, N), float("nan"), device=dev, dtype=torch.float32)
        chain.run_bmm_chain(a, b, c, f, "relu", tile_variant=variant, relu_out=True)
        torch.cuda.synchronize()
        got = f.cpu().numpy()
        assert (got >= 0).all() and (got == 0).mean() > 0.2
        mx, rel = errors(got, want)
        assert mx <= MAX_ABS and rel <= REL_L2, (variant, mx, rel)
    with pytest.raises(NotImplementedError):  # no such slot behind the softmax chain
        chain.run_bmm_chain(a.half(), b.half(), c.half(), torch.empty(batch, M, N, device=dev, dtype=torch.float16),
                            "softmax", relu_out=True)
