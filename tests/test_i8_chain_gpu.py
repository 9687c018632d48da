"""Bit-exact parity of the int8 requantised GEMM chain against the exact-integer checker."""
import numpy as np
import pytest
import torch

from ditto_amd import chain

pytestmark = pytest.mark.gpu


def run_i8(A, B, D, scale=None, uniform=None):
    dev = "cuda:0"
    a, b, d = (torch.from_numpy(np.ascontiguousarray(x)).to(dev) for x in (A, B, D))
    M, N = A.shape[-2], D.shape[-1]
    shape = (A.shape[0], M, N) if A.ndim == 3 else (M, N)
    e = torch.full(shape, -7, dtype=torch.int32, device=dev)
    aux = None if scale is None else torch.from_numpy(scale).to(dev)
    chain.run_bmm_chain(a, b, d, e, "requant", requant_scale=uniform if uniform is not None else 1.0, aux=aux)
    torch.cuda.synchronize()
    return e.cpu().numpy()


@pytest.mark.parametrize("shape", [
    # M, K, L, N
    (64, 64, 256, 256),
    (128, 128, 256, 512),
    (100, 96, 48, 80),       # ragged M, L below one chunk, N below one chunk
    (200, 1024, 256, 1024),  # the full K / L / N of the quantised configuration, fewer rows
    (64, 64, 512, 272),      # two L chunks
    (37, 16, 16, 16),        # smallest legal extents
])
def test_i8_chain_bit_exact(oracle, shape):
    M, K, L, N = shape
    A, B, D, scale = oracle.make_i8_chain_inputs(M, K, L, N, seed=M + N)
    want = oracle.gemm_chain_i8(A, B, D, scale)[0]
    got = run_i8(A, B, D, scale)
    assert got.dtype == np.int32 and np.array_equal(got, want)
    # uniform scale through the descriptor gives the same result as the vector
    assert np.array_equal(run_i8(A, B, D, None, uniform=2.0 ** -10), want)


@pytest.mark.parametrize("shape", [(64, 64, 256, 256), (100, 96, 48, 80), (200, 1024, 256, 1024), (37, 16, 16, 16)])
@pytest.mark.parametrize("relu", [False, True])
def test_i8_wrapping_chain_bit_exact(oracle, shape, relu):
    """The reference's own int8 chain: the middle result (and, with an int8 output, the result) keeps the low byte
    of its int32 accumulator (bmm_bmm_cuda.py:116, :147), optionally behind a ReLU."""
    M, K, L, N = shape
    A, B, D, _ = oracle.make_i8_chain_inputs(M, K, L, N, seed=M + N + 1)
    want, mid = oracle.gemm_chain_i8_wrap(A, B, D, relu, return_mid=True)
    assert (np.abs(A.astype(np.int64) @ B.astype(np.int64)) > 127).any()  # the wrap is exercised
    dev = "cuda:0"
    a, b, d = (torch.from_numpy(np.ascontiguousarray(x)).to(dev) for x in (A, B, D))
    e32 = torch.full((M, N), -7, dtype=torch.int32, device=dev)
    chain.run_bmm_chain(a, b, d, e32, "relu" if relu else "cast")
    e8 = torch.full((M, N), -7, dtype=torch.int8, device=dev)
    chain.run_bmm_chain(a, b, d, e8, "relu" if relu else "cast")
    torch.cuda.synchronize()
    assert np.array_equal(e32.cpu().numpy(), want[0])
    assert np.array_equal(e8.cpu().numpy(), want[0].astype(np.int8))  # numpy's cast keeps the low byte too


def test_i8_chain_variants_agree(oracle):
    """Every kernel variant (32 or 64 rows per workgroup, ring depth) can be forced and gives the same bits."""
    M, K, L, N = 300, 256, 256, 512
    A, B, D, scale = oracle.make_i8_chain_inputs(M, K, L, N, seed=9)
    want = oracle.gemm_chain_i8(A, B, D, scale)[0]
    dev = "cuda:0"
    a, b, d = (torch.from_numpy(np.ascontiguousarray(x)).to(dev) for x in (A, B, D))
    aux = torch.from_numpy(scale).to(dev)
    for variant in (8012, 8014, 8022, 8023):
        e = torch.full((M, N), -7, dtype=torch.int32, device=dev)
        desc = chain.bmm_chain_desc(a, b, d, e, "requant", tile_variant=variant)
        assert chain.select_tile(desc).variant == variant
        chain.run_bmm_chain(a, b, d, e, aux=aux, desc=desc)
        torch.cuda.synchronize()
        assert np.array_equal(e.cpu().numpy(), want), variant
    with pytest.raises(ValueError):
        chain.bmm_chain_desc(a, b, d, e, "requant", tile_variant=8013) and chain.select_tile(
            chain.bmm_chain_desc(a, b, d, e, "requant", tile_variant=8013))


def test_i8_chain_per_column_scales_and_saturation(oracle):
    M, K, L, N = 96, 256, 64, 48
    A, B, D, _ = oracle.make_i8_chain_inputs(M, K, L, N, seed=5)
    rng = np.random.default_rng(1)
    scale = (2.0 ** -rng.integers(6, 14, L)).astype(np.float32)
    scale[::7] = np.float32(0.0123)  # not a power of two: exercises the fp32 multiply + RNE
    want, mid = oracle.gemm_chain_i8(A, B, D, scale, return_mid=True)
    assert (mid == 127).any() and (mid == -128).any()  # both saturation ends are hit
    assert np.array_equal(run_i8(A, B, D, scale), want[0])


def test_i8_chain_ties_round_to_even(oracle):
    # A = row of ones times B = multiples of 512 gives exact .5 ties at scale 2^-10
    M, K, L, N = 64, 16, 16, 16
    A = np.zeros((M, K), np.int8); A[:, 0] = 1
    B = np.zeros((K, L), np.int8)
    D = np.eye(L, N, dtype=np.int8)
    A[:, 1] = 4; B[1, :] = 127          # 508
    A[:, 2] = 4; B[2, :] = np.arange(1, 17)  # 4*(1..16): with 508 -> 512, 516, ...
    scale = np.full(L, 2.0 ** -10, np.float32)
    want = oracle.gemm_chain_i8(A, B, D, scale)[0]
    got = run_i8(A, B, D, scale)
    assert np.array_equal(got, want)
    assert got[0, 0] == 0  # 512 / 1024 = 0.5 rounds to even 0


def test_i8_chain_batched_and_full_rows(oracle):
    rng = np.random.default_rng(2)
    batch, M, K, L, N = 3, 70, 64, 32, 64
    A = rng.integers(-127, 128, (batch, M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (batch, K, L), dtype=np.int8)
    D = rng.integers(-127, 128, (batch, L, N), dtype=np.int8)
    scale = np.full(L, 2.0 ** -9, np.float32)
    want = oracle.gemm_chain_i8(A, B, D, scale)
    assert np.array_equal(run_i8(A, B, D, scale), want)


def test_i8_chain_full_size_properties(oracle):
    # BASELINE size: A[8192,1024], B[1024,256], D[256,1024].  The exact oracle runs on a row
    # sample; the whole output is checked through linearity in D: E(D1 + D2) = E(D1) + E(D2)
    M, K, L, N = 8192, 1024, 256, 1024
    A, B, D, scale = oracle.make_i8_chain_inputs(M, K, L, N, seed=0)
    got = run_i8(A, B, D, scale)
    rows = np.r_[0:64, 4000:4064, 8128:8192]
    want = oracle.gemm_chain_i8(A[rows], B, D, scale)[0]
    assert np.array_equal(got[rows], want)
    D1 = (D // 2).astype(np.int8)
    D2 = (D - D1).astype(np.int8)
    assert np.array_equal(run_i8(A, B, D1, scale) + run_i8(A, B, D2, scale), got)


def test_i8_chain_rejects_bad_descriptors():
    dev = "cuda:0"
    a = torch.zeros(64, 64, dtype=torch.int8, device=dev)
    b = torch.zeros(64, 32, dtype=torch.int8, device=dev)
    d = torch.zeros(32, 64, dtype=torch.int8, device=dev)
    e = torch.zeros(64, 64, dtype=torch.int32, device=dev)
    with pytest.raises(NotImplementedError):
        chain.run_bmm_chain(a, b, d, e, "softmax")
    with pytest.raises(ValueError):
        chain.run_bmm_chain(a[:, :60], b[:60], d, e, "requant")
    with pytest.raises(ValueError):
        chain.run_bmm_chain(a, b, d, e, "requant", aux=torch.ones(5, device=dev))
    with pytest.raises(ValueError):
        chain.run_bmm_chain(a, b, d, e.float(), "requant")


def test_i8_chain_through_the_operator_api(oracle):
    """The quantised configuration (int8 A[8192,1024], B[1024,256], D[256,1024], middle result requantised
    at 2^-10) built the way the reference builds its chains -- BatchGemmGemm -> serial fusion state ->
    build_fusion_choice -> tensorize_cuda -> build -> f(A, B, D, E) -- and checked bit for bit."""
    import ditto_amd as ditto
    from ditto_amd import auto_compute as ac, auto_tensorize as at, hardware as hw

    def built(ins, outs):
        layer = ac.layer([outs[0].op], inputs=list(ins))
        sfs = at.build_serial_fusion_state(layer)
        packed = at.cuda_wmma(16, 16, 16, "int8", "int32", "global")
        infos = {op: at.match_info(at.intrinsic_match(op.output(0), packed, ["InnerMost", "SameRange"])[0], packed)
                 for op in (sfs.first_op, sfs.second_op)}
        sfs.register_tensorize_axes([iv for mi in infos.values() for iv in mi.axis])
        fc = at.build_fusion_choice(sfs, hw.query_hw_param("gpu.hip.MI355X"), "int32")
        state = at.tensorize_hyper_fusion_state(layer, fc, infos)
        sch = at.tensorize_cuda(layer, state, hw.query_hw_param("gpu.hip.MI355X"), at.cuda_tensorize_param())
        return ditto.build(sch, layer.schedule_tensors, "hip")

    dev = "cuda:0"
    M, K, L, N = 8192, 1024, 256, 1024
    A, B, D, scale = oracle.make_i8_chain_inputs(M, K, L, N, seed=11)
    func = built(*ac.nn.functional.BatchGemmGemm(1, M, N, K, L, "int8", "int32", requant_scale=2.0 ** -10))
    a, b, d = (torch.from_numpy(x[None]).to(dev) for x in (A, B, D))
    e = torch.full((1, M, N), -7, dtype=torch.int32, device=dev)
    func(a, b, d, e)
    torch.cuda.synchronize()
    got = e.cpu().numpy()[0]
    rows = np.r_[0:64, 4000:4100, M - 37:M]  # rows are independent: the checker runs on a sample of them
    want = oracle.gemm_chain_i8(A[rows], B, D, scale)[0]
    assert np.array_equal(got[rows], want)
    assert np.array_equal(got, run_i8(A, B, D, scale))  # and all of it equals the direct C-ABI call
    # per-column scales as a fourth input tensor
    M2, K2, L2, N2 = 96, 256, 64, 48
    A2, B2, D2, _ = oracle.make_i8_chain_inputs(M2, K2, L2, N2, seed=5)
    sc = (2.0 ** -np.random.default_rng(1).integers(6, 14, L2)).astype(np.float32)
    func2 = built(*ac.nn.functional.BatchGemmGemm(1, M2, N2, K2, L2, "int8", "int32", scale_tensor=True))
    e2 = torch.zeros((1, M2, N2), dtype=torch.int32, device=dev)
    func2(*(torch.from_numpy(x[None]).to(dev) for x in (A2, B2, D2)), torch.from_numpy(sc).to(dev), e2)
    torch.cuda.synchronize()
    assert np.array_equal(e2.cpu().numpy()[0], oracle.gemm_chain_i8(A2, B2, D2, sc)[0])
