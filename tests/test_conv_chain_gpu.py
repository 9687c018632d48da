"""GPU parity of the fused conv -> conv chain against the CPU checker (NCHW, fp16 / bf16)."""
import numpy as np
import pytest
import torch

from ditto_amd import chain
from tests.gpu_util import errors, report, to_dev, TORCH_DTYPES

pytestmark = pytest.mark.gpu

# fp16 and bf16 alike against the checker that rounds the intermediate and the output where the chain does
# (bf16 measured: at most 1.1e-4 rel-L2, from roundings that flip on the last accumulator bits)
MAX_ABS, REL_L2 = 1e-2, 1e-3


def run_conv(X, W1, W2, dtype, pad1=1, stride1=1, inter="cast", relu_out=False, out_dtype=None, workspace=None,
             pad2=0, groups1=1, tile_variant=0, stride2=1):
    x, w1, w2 = to_dev(X, dtype), to_dev(W1, dtype), to_dev(W2, dtype)
    N, _, H, W = X.shape
    R, S = W1.shape[2:]
    P = ((H + 2 * pad1 - R) // stride1 + 1 + 2 * pad2 - W2.shape[2]) // stride2 + 1
    Q = ((W + 2 * pad1 - S) // stride1 + 1 + 2 * pad2 - W2.shape[3]) // stride2 + 1
    y = torch.full((N, W2.shape[0], P, Q), float("nan"), device=x.device, dtype=TORCH_DTYPES[out_dtype or dtype])
    chain.run_conv_chain(x, w1, w2, y, pad1, stride1, pad2, stride2, inter, relu_out, workspace=workspace,
                         groups1=groups1, tile_variant=tile_variant)
    torch.cuda.synchronize()
    return y.float().cpu().numpy()


CASES = [
    # N, C0, H, W, C1, R, pad, stride, C2
    (2, 64, 56, 56, 64, 3, 1, 1, 256),   # the chain of the workload definition, 2 images
    (1, 16, 12, 20, 32, 3, 1, 1, 40),    # small, C2 not a multiple of 32
    (2, 24, 17, 23, 64, 3, 1, 2, 64),    # odd extents, stride 2, C0 not a multiple of 16
    (1, 64, 28, 28, 128, 3, 1, 1, 64),   # Darknet-19 row of the reference's table (scaled down)
    (1, 32, 14, 14, 256, 3, 1, 1, 128),  # 256 intermediate channels
    (2, 64, 56, 56, 64, 1, 0, 1, 64),    # conv1x1 -> conv1x1 (modified ResNet-50 row)
    (1, 8, 9, 140, 16, 3, 1, 1, 16),     # wider than one tile
    (1, 16, 30, 30, 24, 5, 2, 1, 32),    # 5x5 first filter, C1 padded to 32
]


def rows_pipeline_shape(case):
    """3x3 (pad 1, stride 1) -> 1x1, at most 64 -> 64 -> 256 channels, rows of whole 16-byte vectors up to 64 pixels:
    with a 16-bit output and a workspace these run on the row pipeline."""
    N, C0, H, W, C1, R, pad, stride, C2 = case
    fits = R == 3 and pad == 1 and stride == 1 and C0 <= 64 and C1 <= 64 and C2 <= 256 and W % 8 == 0 and W <= 64
    # ... and where it pays: more than 32 channels somewhere before the output, and a wide output or few images
    rows_per_tile = max(1, 256 // W)
    return fits and max(C0, C1) > 32 and (C2 >= 192 or N * -(-H // rows_per_tile) < 256)


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_conv_chain_vs_oracle(oracle, case, dtype):
    N, C0, H, W, C1, R, pad, stride, C2 = case
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, R, 1, dtype, seed=C0 + C1, w_std=0.05)
    want32 = oracle.conv_chain_f32(X, W1, W2, pad, stride, 0, 1, round_mid=dtype)
    # with the repacked-weights workspace (None: the wrapper's cached buffer) and without (False)
    for ws in (None, False):
        got32 = run_conv(X, W1, W2, dtype, pad, stride, out_dtype="float32", workspace=ws)
        assert np.isfinite(got32).all(), ws
        mx, rel = errors(got32, want32)
        assert mx <= MAX_ABS and rel <= REL_L2, (ws, mx, rel)
        got = run_conv(X, W1, W2, dtype, pad, stride, workspace=ws)
        if not (ws is None and rows_pipeline_shape(case)):
            # (with a workspace that shape runs on the row pipeline, whose summation order is its own)
            assert np.array_equal(got, oracle.np_round_to(got32, dtype)), ws
        mx, rel = errors(got, oracle.np_round_to(want32, dtype))
        if dtype == "bfloat16":
            report("conv chain bf16 %s" % (case,), mx, rel)
        assert mx <= MAX_ABS and rel <= REL_L2, (ws, mx, rel)


CASES_ROWS_PIPELINE = [
    # N, C0, H, W, C1, C2: conv3x3 (pad 1, stride 1) -> conv1x1 on the row pipeline
    (2, 64, 56, 56, 64, 256),   # the workload's shape, 2 images: bands of 7 rows (3 steps of two rows and one of one)
    (1, 64, 9, 64, 64, 256),    # the widest row (two full pixel tiles, 16 strips per step); bands of 5
    (3, 24, 11, 8, 40, 72),     # one strip per row, channel counts that fill no tile, a short last band
    (1, 16, 1, 16, 40, 16),     # a single output row
    (2, 48, 30, 40, 32, 136),   # the third store wave takes 8 of its 64 channels, the fourth none
    (40, 8, 12, 24, 48, 32),    # many images of few rows
]


@pytest.mark.parametrize("case", CASES_ROWS_PIPELINE)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_conv_chain_row_pipeline(oracle, case, dtype):
    """The row pipeline against the oracle and against the general kernel on the same inputs (different
    summation orders: held to the workload tolerance), through run and through prepare + run_prepared."""
    N, C0, H, W, C1, C2 = case
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, 3, 1, dtype, seed=C0 + C2 + W, w_std=0.05)
    x, w1, w2 = to_dev(X, dtype), to_dev(W1, dtype), to_dev(W2, dtype)
    for relu in (False, True):
        inter = "relu" if relu else "cast"
        y = torch.full((N, C2, H, W), float("nan"), device=x.device, dtype=x.dtype)
        desc = chain.conv_chain_desc(x, w1, w2, y, 1, 1, 0, 1, inter, relu)
        assert chain.select_tile(desc).variant // 100 == 37
        chain.run_conv_chain(x, w1, w2, y, desc=desc)
        torch.cuda.synchronize()
        got = y.float().cpu().numpy()
        assert np.isfinite(got).all()
        want = oracle.conv_chain_f32(X, W1, W2, 1, 1, 0, 1, relu_mid=relu, relu_out=relu, round_mid=dtype)
        mx, rel = errors(got, oracle.np_round_to(want, dtype))
        if dtype == "bfloat16" and relu:
            report("conv chain bf16 row pipeline %s" % (case,), mx, rel)
        assert mx <= MAX_ABS and rel <= REL_L2, (relu, mx, rel)
        # prepared weights: same bits as the one-call form
        ws = chain.prepare_conv_chain(desc, w1, w2)
        y1 = torch.full_like(y, float("nan"))
        chain.run_conv_chain(x, w1, w2, y1, desc=desc, workspace=ws, prepared=True)
        torch.cuda.synchronize()
        assert torch.equal(y1, y), relu
        y2 = torch.full_like(y, float("nan"))
        desc2 = chain.conv_chain_desc(x, w1, w2, y2, 1, 1, 0, 1, inter, relu, tile_variant=3000)  # the general kernel
        assert chain.select_tile(desc2).variant // 100 in (30, 31)
        chain.run_conv_chain(x, w1, w2, y2, desc=desc2)
        torch.cuda.synchronize()
        mx, rel = errors(got, y2.float().cpu().numpy())
        assert mx <= MAX_ABS and rel <= REL_L2, (relu, mx, rel)


# Enough tiles of whole output rows for two rounds of persistent workgroups (at least 512), 16-bit
# output, at most 64 input / intermediate channels: the opt-in kernel with both weight tensors resident
# on the CU (tile_variant 3900).
CASES_PERSISTENT = [
    # N, C0, H, W, C1, R, pad, stride, C2
    (520, 8, 8, 8, 16, 3, 1, 1, 32),      # one tile per image, 32-channel variants
    (130, 40, 26, 16, 48, 3, 1, 1, 200),  # padded channels in every tensor; last tile of an image partial
    (64, 64, 32, 32, 64, 3, 1, 1, 256),   # the largest weights: 64 -> 64 (3x3) -> 256
    (128, 64, 33, 32, 64, 3, 1, 2, 128),  # stride 2, 17 x 16 output: two staging tasks per thread
    (96, 16, 24, 48, 32, 1, 0, 1, 96),    # conv1x1 -> conv1x1, two rows of 48 per tile
    (260, 24, 19, 32, 64, 3, 1, 2, 64),   # stride 2, 10 x 16 output, 8-row tiles
]


PERSIST_OFF = ("the persistent conv chain kernel is switched off in the planner (DITTO_EUNSUPPORTED): it waits for "
               "prefetch loads the compiler does not track with a hand-counted s_waitcnt and is slower than the default")


@pytest.mark.skip(reason=PERSIST_OFF)
@pytest.mark.parametrize("case", CASES_PERSISTENT)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_persistent_conv_chain_vs_oracle(oracle, case, dtype):
    N, C0, H, W, C1, R, pad, stride, C2 = case
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, R, 1, dtype, seed=C0 + C2, w_std=0.05)
    x, w1, w2 = to_dev(X, dtype), to_dev(W1, dtype), to_dev(W2, dtype)
    P, Q = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - R) // stride + 1
    y = torch.empty((N, C2, P, Q), device=x.device, dtype=TORCH_DTYPES[dtype])
    desc = chain.conv_chain_desc(x, w1, w2, y, pad, stride, 0, 1, "cast", False, tile_variant=3900)
    assert chain.select_tile(desc).variant // 100 == 39  # the persistent kernel
    for relu in (False, True):
        want32 = oracle.conv_chain_f32(X, W1, W2, pad, stride, 0, 1, relu_mid=relu, relu_out=relu, round_mid=dtype)
        got = run_conv(X, W1, W2, dtype, pad, stride, "relu" if relu else "cast", relu, tile_variant=3900)
        assert got.shape == want32.shape and np.isfinite(got).all()
        mx, rel = errors(got, oracle.np_round_to(want32, dtype))
        assert mx <= MAX_ABS and rel <= REL_L2, (relu, mx, rel)
        # against the one-tile-per-workgroup kernel (taken when there is no workspace); their summation
        # orders differ (here two waves each sum half of the taps x channel groups)
        other = run_conv(X, W1, W2, dtype, pad, stride, "relu" if relu else "cast", relu, workspace=False)
        assert errors(got, other)[1] <= REL_L2, relu
    # a second call right away (the halo prefetch and the stores of the first are independent of it)
    again = run_conv(X, W1, W2, dtype, pad, stride, "relu", True)
    assert np.array_equal(again, got)


CASES_3X3_SECOND = [
    # N, C0, H, W, C1, R1, pad1, stride1, C2, R2, pad2
    (2, 64, 56, 56, 64, 1, 0, 1, 64, 3, 1),    # conv1x1 -> conv3x3 (conv1x1_conv3x3_cuda.py:77-189)
    (1, 32, 20, 28, 32, 1, 0, 1, 72, 3, 1),    # C2 not a multiple of 64
    (1, 16, 33, 45, 64, 1, 0, 2, 32, 3, 1),    # strided 1x1 first, odd extents
    (1, 32, 18, 18, 32, 3, 1, 1, 48, 3, 1),    # conv3x3 -> conv3x3
    (1, 16, 12, 150, 16, 1, 0, 1, 16, 3, 1),   # wider than one tile
    (1, 16, 16, 16, 32, 3, 1, 1, 32, 3, 0),    # unpadded second convolution
    (2, 24, 30, 30, 64, 3, 1, 1, 128, 3, 1),   # conv3x3 -> conv3x3, 64 intermediate channels, C0 % 32 != 0
    # 1x1 -> 3x3 with rows of whole 16-byte vectors and at most 64 channels: the persistent kernel with W2 in LDS
    (1, 32, 21, 24, 48, 1, 0, 1, 40, 3, 1),    # channel counts that are no multiples of 32; a partial last tile
    (1, 8, 9, 8, 8, 1, 0, 1, 8, 3, 1),         # one small tile
    (3, 64, 7, 128, 16, 1, 0, 1, 64, 3, 1),    # two output rows per tile
    # more than 64 intermediate channels (general kernel, four tiles of 32)
    (1, 32, 20, 24, 128, 1, 0, 1, 64, 3, 1),   # conv1x1 -> conv3x3, 128 intermediate channels
    (1, 16, 14, 14, 96, 3, 1, 1, 40, 3, 1),    # conv3x3 -> conv3x3, 96 intermediate channels
]


def rows13_shape(N, C0, W, C1, R1, pad1, stride1, C2, R2, pad2):
    """1x1 -> 3x3 (pad 1), at most 64 channels everywhere, rows of whole 16-byte vectors up to 64 pixels: with a
    16-bit output these run on the row pipeline with the 1x1 convolution in its transposing stage."""
    return (R1 == 1 and pad1 == 0 and stride1 == 1 and R2 == 3 and pad2 == 1 and max(C0, C1, C2) <= 64 and
            C0 % 8 == 0 and W % 8 == 0 and W <= 64)


@pytest.mark.parametrize("case", CASES_3X3_SECOND)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_conv_chain_with_wide_second_filter(oracle, case, dtype):
    N, C0, H, W, C1, R1, pad1, stride1, C2, R2, pad2 = case
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, R1, R2, dtype, seed=C0 + C2, w_std=0.05)
    for relu in (False, True):
        want32 = oracle.conv_chain_f32(X, W1, W2, pad1, stride1, pad2, 1, relu_mid=relu, relu_out=relu, round_mid=dtype)
        got32 = run_conv(X, W1, W2, dtype, pad1, stride1, "relu" if relu else "cast", relu, "float32", None, pad2)
        assert got32.shape == want32.shape and np.isfinite(got32).all()
        mx, rel = errors(got32, want32)
        assert mx <= MAX_ABS and rel <= REL_L2, (relu, mx, rel)
    got = run_conv(X, W1, W2, dtype, pad1, stride1, "relu", True, None, None, pad2)
    if rows13_shape(N, C0, W, C1, R1, pad1, stride1, C2, R2, pad2):
        # (with a 16-bit output that shape runs on the row pipeline, whose summation order is its own)
        mx, rel = errors(got, oracle.np_round_to(want32, dtype))
        assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)
    else:
        assert np.array_equal(got, oracle.np_round_to(got32, dtype))
    with pytest.raises(ValueError):  # this variant cannot run without its workspace
        run_conv(X, W1, W2, dtype, pad1, stride1, workspace=False, pad2=pad2)


CASES_ROWS13 = [
    # N, C0, H, W, C1, C2
    (2, 64, 56, 56, 64, 64),    # the reference's ResNet-50 row (conv1x1_conv3x3_cuda.py:348-350), 2 images
    (1, 32, 21, 24, 48, 40),    # channel counts that are no multiples of 32, an odd number of rows, one pixel tile
    (1, 8, 9, 8, 8, 8),         # the smallest rows
    (3, 16, 7, 64, 64, 24),     # the widest rows; fewer output channels than one store wave's 16 times two
    (1, 64, 5, 40, 32, 64),     # two pixel tiles, the second one partial
    (40, 24, 30, 48, 56, 16),   # more bands than CUs; only the first store wave has channels
    (1, 40, 1, 16, 64, 64),     # a single image row
]


@pytest.mark.parametrize("case", CASES_ROWS13)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_row_pipeline_conv1x1_conv3x3(oracle, case, dtype):
    """conv1x1 -> conv3x3 (pad 1) through the row pipeline: against the oracle, and against the kernel that keeps
    W2 in LDS on the same inputs."""
    N, C0, H, W, C1, C2 = case
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, 1, 3, dtype, seed=C0 + C2 + H, w_std=0.05)
    x, w1, w2 = to_dev(X, dtype), to_dev(W1, dtype), to_dev(W2, dtype)
    y = torch.empty((N, C2, H, W), device=x.device, dtype=TORCH_DTYPES[dtype])
    tile = chain.select_tile(chain.conv_chain_desc(x, w1, w2, y, 0, 1, 1, 1, "relu", False))
    assert tile.variant // 100 == 38 and tile.block_threads == 512 and tile.lds_bytes <= 160 * 1024
    for relu_mid, relu_out in ((False, False), (True, False), (False, True), (True, True)):
        inter = "relu" if relu_mid else "cast"
        want = oracle.np_round_to(oracle.conv_chain_f32(X, W1, W2, 0, 1, 1, 1, relu_mid=relu_mid, relu_out=relu_out,
                                                        round_mid=dtype), dtype)
        got = run_conv(X, W1, W2, dtype, 0, 1, inter, relu_out, None, None, 1)
        assert got.shape == want.shape and np.isfinite(got).all()
        mx, rel = errors(got, want)
        assert mx <= MAX_ABS and rel <= REL_L2, (relu_mid, relu_out, mx, rel)
        again = run_conv(X, W1, W2, dtype, 0, 1, inter, relu_out, None, None, 1)
        assert np.array_equal(again, got)
    # prepared weights: same bits as the one-call form; without the workspace the prepared form is refused
    desc = chain.conv_chain_desc(x, w1, w2, y, 0, 1, 1, 1, "relu", True)
    ws = chain.prepare_conv_chain(desc, w1, w2)
    y1 = torch.full_like(y, float("nan"))
    chain.run_conv_chain(x, w1, w2, y1, desc=desc, workspace=ws, prepared=True)
    torch.cuda.synchronize()
    assert np.array_equal(y1.float().cpu().numpy(), got)
    # a 1x1 weight tensor that is only element-aligned: the one-call form runs the general kernel instead
    w1_off = torch.empty(w1.numel() + 1, device=x.device, dtype=w1.dtype)[1:].view_as(w1).copy_(w1)
    assert w1_off.data_ptr() % 16 != 0
    y3 = torch.full_like(y, float("nan"))
    chain.run_conv_chain(x, w1_off, w2, y3, 0, 1, 1, 1, "relu", True)
    torch.cuda.synchronize()
    mx, rel = errors(y3.float().cpu().numpy(), got)
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)
    with pytest.raises(ValueError):  # ... and the prepared form, whose weights are in this kernel's layout, reports it
        chain.run_conv_chain(x, w1_off, w2, y3, desc=desc, workspace=ws, prepared=True)
    assert chain.select_tile(chain.conv_chain_desc(x, w1, w2, y, 0, 1, 1, 1, "relu", False,
                                                   tile_variant=3600)).variant // 100 == 36
    other = run_conv(X, W1, W2, dtype, 0, 1, "relu", True, None, None, 1, tile_variant=3600)
    mx, rel = errors(got, other)
    # a forced kernel does not step aside: the element-aligned weights are refused
    with pytest.raises(ValueError):
        chain.run_conv_chain(x, w1_off, w2, y3, 0, 1, 1, 1, "relu", True, tile_variant=3800)
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)


def test_row_pipeline_conv1x1_conv3x3_at_benchmark_size(oracle):
    """The benchmark's shape, 32 x 64 x 56 x 56 -> 64 -> 64 (one band per CU): three images against the oracle, all
    of them against the kernel that keeps W2 in LDS, and the chain's linearity in x (no ReLU: f(2x) = 2 f(x); a power
    of two only shifts exponents, so the two differ only where an intermediate value is subnormal in fp16)."""
    N, C0, H, W, C1, C2 = 32, 64, 56, 56, 64, 64
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, 1, 3, "float16", seed=77, w_std=0.05)
    x, w1, w2 = to_dev(X, "float16"), to_dev(W1, "float16"), to_dev(W2, "float16")
    y = torch.full((N, C2, H, W), float("nan"), device=x.device, dtype=torch.float16)
    desc = chain.conv_chain_desc(x, w1, w2, y, 0, 1, 1, 1, "relu", True)
    assert chain.select_tile(desc).variant == 3807
    chain.run_conv_chain(x, w1, w2, y, desc=desc)
    torch.cuda.synchronize()
    got = y.float().cpu().numpy()
    assert np.isfinite(got).all()
    for n in (0, 17, 31):
        want = oracle.conv_chain_f32(X[n:n + 1], W1, W2, 0, 1, 1, 1, relu_mid=True, relu_out=True, round_mid="float16")
        mx, rel = errors(got[n:n + 1], oracle.np_round_to(want, "float16"))
        assert mx <= MAX_ABS and rel <= REL_L2, (n, mx, rel)
    ya, yb = torch.empty_like(y), torch.empty_like(y)
    chain.run_conv_chain(x, w1, w2, ya, 0, 1, 1, 1, "cast", False)
    chain.run_conv_chain(x * 2, w1, w2, yb, 0, 1, 1, 1, "cast", False)
    torch.cuda.synchronize()
    mx, rel = errors((ya * 2).float().cpu().numpy(), yb.float().cpu().numpy())
    assert mx <= 1e-3 and rel <= 1e-5, (mx, rel)
    y2 = torch.full_like(y, float("nan"))
    desc2 = chain.conv_chain_desc(x, w1, w2, y2, 0, 1, 1, 1, "relu", True, tile_variant=3600)
    assert chain.select_tile(desc2).variant // 100 == 36
    chain.run_conv_chain(x, w1, w2, y2, desc=desc2)
    torch.cuda.synchronize()
    mx, rel = errors(got, y2.float().cpu().numpy())
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)


def test_resident_conv_chain_over_several_rounds(oracle):
    """More tiles than CUs: every persistent workgroup walks over more than one tile.  Checked against the
    general kernel (which streams W2 per workgroup) on the same inputs, both against the oracle on a slice."""
    N, C0, H, W, C1, C2 = 20, 64, 56, 56, 64, 64
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, 1, 3, "float16", seed=5, w_std=0.05)
    x, w1, w2 = to_dev(X, "float16"), to_dev(W1, "float16"), to_dev(W2, "float16")
    y = torch.full((N, C2, H, W), float("nan"), device=x.device, dtype=torch.float16)
    desc = chain.conv_chain_desc(x, w1, w2, y, 0, 1, 1, 1, "relu", False, tile_variant=3600)  # (0: the row pipeline)
    tile = chain.select_tile(desc)
    assert tile.variant == 3604 and tile.block_threads == 512 and tile.lds_bytes <= 160 * 1024
    chain.run_conv_chain(x, w1, w2, y, desc=desc)
    torch.cuda.synchronize()
    got = y.float().cpu().numpy()
    assert np.isfinite(got).all()
    y2 = torch.full_like(y, float("nan"))
    desc2 = chain.conv_chain_desc(x, w1, w2, y2, 0, 1, 1, 1, "relu", False, tile_variant=3500)
    assert chain.select_tile(desc2).variant // 100 == 35
    chain.run_conv_chain(x, w1, w2, y2, desc=desc2)
    torch.cuda.synchronize()
    mx, rel = errors(got, y2.float().cpu().numpy())
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)
    for n in (0, 13, 19):  # first, a middle and the last image (the last one is the second tile of its workgroup)
        want = oracle.conv_chain_f32(X[n:n + 1], W1, W2, 0, 1, 1, 1, relu_mid=True, relu_out=False, round_mid="float16")
        mx, rel = errors(got[n:n + 1], want)
        assert mx <= MAX_ABS and rel <= REL_L2, (n, mx, rel)


CASES_DEPTHWISE = [
    # N, C0, H, W, factor, R, pad, stride, C2
    (1, 32, 56, 56, 16, 3, 1, 1, 64),    # depthwise3x3_conv1x1_small_channel_cuda.py:340-346, row 2
    (2, 16, 40, 40, 16, 3, 1, 2, 32),    # stride 2 (row 4, scaled down)
    (1, 24, 17, 23, 8, 3, 1, 1, 40),     # odd extents, C2 not a multiple of 32, factor 8
    (1, 40, 14, 14, 1, 3, 1, 1, 96),     # plain depthwise (factor 1), MobileNet block
    (1, 12, 9, 300, 2, 3, 1, 1, 16),     # factor 2, wider than one tile, C1 = 24
    (1, 6, 20, 20, 4, 3, 0, 1, 160),     # factor 4, no padding, 256-wide output tile set
    (1, 64, 28, 28, 16, 3, 1, 1, 128),   # 1024 intermediate channels in several chunks
    (1, 8, 12, 12, 24, 2, 0, 1, 32),     # 2x2 filter, factor 24
    (1, 8, 12, 12, 48, 4, 1, 1, 32),     # 4x4 filter (16 taps), factor 48
    (2, 6, 13, 21, 32, 2, 1, 1, 72),     # 2x2 filter (no second tap group), factor 32
    (6, 16, 112, 112, 16, 3, 1, 1, 32),  # more pixel tiles than persistent workgroups: several rounds
    (1, 16, 30, 30, 16, 3, 1, 1, 256),   # 256 output channels; image rows of 30: 4-byte halo loads
    (1, 16, 21, 23, 32, 3, 1, 1, 64),    # odd image rows: 2-byte halo loads, 2-byte output stores
    (1, 48, 24, 24, 16, 3, 1, 2, 64),    # stride 2, 768 intermediate channels
    # output rows that are multiples of 8 with factor 1, 2, 4, 8: the persistent kernel with the
    # depthwise stage on the vector ALU
    (2, 32, 24, 24, 1, 3, 1, 1, 64),     # plain depthwise, MobileNet v1 block
    (1, 40, 16, 16, 1, 3, 1, 1, 96),     # 40 channels: the last block of 32 is partly padding
    (1, 16, 16, 40, 2, 3, 1, 1, 48),     # factor 2
    (1, 8, 32, 32, 4, 3, 1, 2, 32),      # factor 4, stride 2
    (1, 12, 16, 16, 8, 3, 1, 1, 128),    # factor 8, 96 intermediate channels
    (8, 16, 96, 96, 1, 3, 1, 1, 32),     # more tiles than persistent workgroups
    (1, 128, 8, 8, 2, 3, 1, 1, 256),     # 256 output channels
]
DW_VECTOR_ALU_CASES = [c for c in CASES_DEPTHWISE if c[4] in (1, 2, 4, 8) and ((c[3] + 2 * c[6] - 3) // c[7] + 1) % 8 == 0]
# factor 1, stride 1, at most 32 -> 64 channels, rows of whole 16-byte vectors up to 128 pixels: the
# row-streaming kernel takes these when the output is 16-bit
DW_ROWS_CASES = [c for c in DW_VECTOR_ALU_CASES if c[4] == 1 and c[7] == 1 and c[1] <= 32 and c[8] <= 64 and c[3] <= 128]


@pytest.mark.parametrize("case", CASES_DEPTHWISE)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_depthwise_conv_chain_vs_oracle(oracle, case, dtype):
    N, C0, H, W, factor, R, pad, stride, C2 = case
    C1 = C0 * factor
    rng = np.random.default_rng(C0 + C2)
    X = oracle.np_round_to(rng.standard_normal((N, C0, H, W)).astype(np.float32), dtype)
    W1 = oracle.np_round_to(rng.standard_normal((C1, 1, R, R)).astype(np.float32) * 0.3, dtype)
    W2 = oracle.np_round_to(rng.standard_normal((C2, C1, 1, 1)).astype(np.float32) * 0.05, dtype)
    for relu in (False, True):
        want32 = oracle.conv_chain_f32(X, W1, W2, pad, stride, 0, 1, relu_mid=relu, relu_out=relu, round_mid=dtype,
                                       groups1=C0)
        got32 = run_conv(X, W1, W2, dtype, pad, stride, "relu" if relu else "cast", relu, "float32", groups1=C0)
        assert got32.shape == want32.shape and np.isfinite(got32).all()
        mx, rel = errors(got32, want32)
        assert mx <= MAX_ABS and rel <= REL_L2, (relu, mx, rel)
    got = run_conv(X, W1, W2, dtype, pad, stride, "relu", True, groups1=C0)
    if case in DW_VECTOR_ALU_CASES:
        # fp32 output runs the plain kernel there and 16-bit output the persistent one: their
        # summation orders differ, so the 16-bit result is held to the oracle, not to the fp32 bits
        mx, rel = errors(got, oracle.np_round_to(want32, dtype))
        if dtype == "bfloat16":
            report("conv chain (wide second filter / depthwise) bf16 %s" % (case,), mx, rel)
        assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)
    else:
        assert np.array_equal(got, oracle.np_round_to(got32, dtype))


@pytest.mark.parametrize("case", DW_VECTOR_ALU_CASES)
def test_small_factor_cases_run_the_persistent_kernel(case):
    """The cases meant for it do select the persistent kernel with the vector-ALU depthwise stage
    (variant 4000 + 10 * output-channel tiles + 3), so the parity cases above cover it."""
    N, C0, H, W, factor, R, pad, stride, C2 = case
    dev = "cuda:0"
    x = torch.empty(N, C0, H, W, device=dev, dtype=torch.float16)
    w1 = torch.empty(C0 * factor, 1, R, R, device=dev, dtype=torch.float16)
    w2 = torch.empty(C2, C0 * factor, 1, 1, device=dev, dtype=torch.float16)
    P, Q = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - R) // stride + 1
    y = torch.empty(N, C2, P, Q, device=dev, dtype=torch.float16)
    desc = chain.conv_chain_desc(x, w1, w2, y, pad, stride, 0, 1, "cast", False, C0)
    assert chain.select_tile(desc).variant % 10 == (4 if case in DW_ROWS_CASES else 3)


CASES_DW_ROWS = [
    # N, C0, H, W, C2: depthwise 3x3 (factor 1, pad 1, stride 1) -> 1x1 on the row-streaming kernel
    (2, 32, 112, 112, 64),   # MobileNet-V1's first separable block: 7 load instructions per row, many bands
    (1, 32, 56, 56, 64),     # half-filled last load instruction of a row (224 of 256 lanes)
    (3, 7, 9, 8, 64),        # one strip per row, odd channel count, fewer rows than a band
    (1, 24, 5, 128, 40),     # the widest row; output channels that do not fill their tiles
    (2, 16, 33, 40, 24),     # a last band shorter than the others
    (1, 32, 19, 72, 64),
    (40, 8, 16, 16, 16),     # more workgroups than CUs with many bands
]


@pytest.mark.parametrize("case", CASES_DW_ROWS)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_row_streaming_depthwise_chain(oracle, case, dtype):
    """The row-streaming kernel against the oracle and against the persistent kernel on the same inputs
    (both accumulate in fp32 in different orders: held to the workload tolerance, not to the bits)."""
    N, C0, H, W, C2 = case
    rng = np.random.default_rng(C0 + C2 + W)
    X = oracle.np_round_to(rng.standard_normal((N, C0, H, W)).astype(np.float32), dtype)
    W1 = oracle.np_round_to(rng.standard_normal((C0, 1, 3, 3)).astype(np.float32) * 0.3, dtype)
    W2 = oracle.np_round_to(rng.standard_normal((C2, C0, 1, 1)).astype(np.float32) * 0.2, dtype)
    x, w1, w2 = to_dev(X, dtype), to_dev(W1, dtype), to_dev(W2, dtype)
    for relu in (False, True):
        y = torch.full((N, C2, H, W), float("nan"), device=x.device, dtype=x.dtype)
        desc = chain.conv_chain_desc(x, w1, w2, y, 1, 1, 0, 1, "relu" if relu else "cast", relu, C0)
        assert chain.select_tile(desc).variant == 4024
        chain.run_conv_chain(x, w1, w2, y, desc=desc)
        torch.cuda.synchronize()
        got = y.float().cpu().numpy()
        assert np.isfinite(got).all()
        want = oracle.conv_chain_f32(X, W1, W2, 1, 1, 0, 1, relu_mid=relu, relu_out=relu, round_mid=dtype, groups1=C0)
        mx, rel = errors(got, oracle.np_round_to(want, dtype))
        if dtype == "bfloat16" and relu:
            report("conv chain (wide second filter / depthwise) bf16 rows %s" % (case,), mx, rel)
        assert mx <= MAX_ABS and rel <= REL_L2, (relu, mx, rel)
        y2 = torch.full_like(y, float("nan"))
        desc2 = chain.conv_chain_desc(x, w1, w2, y2, 1, 1, 0, 1, "relu" if relu else "cast", relu, C0, tile_variant=4000)
        assert chain.select_tile(desc2).variant % 10 != 4
        chain.run_conv_chain(x, w1, w2, y2, desc=desc2)
        torch.cuda.synchronize()
        mx, rel = errors(got, y2.float().cpu().numpy())
        assert mx <= MAX_ABS and rel <= REL_L2, (relu, mx, rel)


CASES_DW16_ROWS = [
    # N, C0, H, W, C2: depthwise 3x3 (factor 16, pad 1, stride 1) -> 1x1 on the row-streaming kernel for that factor
    (2, 32, 112, 112, 64),   # the reference's MobileNet row: 49 tiles per band, rows of 15 chunks, ring of 8 rows
    (1, 32, 56, 56, 64),     # tiles that span two image rows; ring of 16 rows
    (3, 6, 9, 24, 40),       # few channels, output channels that do not fill their tiles, a band of every row
    (1, 24, 5, 120, 40),     # the widest row
    (2, 16, 33, 40, 24),     # a last band shorter than the others, a last tile that is not full
    (1, 32, 19, 72, 64),
    (40, 8, 16, 16, 16),     # many small images
]


@pytest.mark.parametrize("case", CASES_DW16_ROWS)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_row_streaming_depthwise_chain_factor_16(oracle, case, dtype):
    """The row-streaming kernel for sixteen outputs per input channel against the oracle and against the tiled
    kernel on the same inputs (the same MFMAs in the same order: the same bits)."""
    N, C0, H, W, C2 = case
    C1 = 16 * C0
    rng = np.random.default_rng(C0 + C2 + W)
    X = oracle.np_round_to(rng.standard_normal((N, C0, H, W)).astype(np.float32), dtype)
    W1 = oracle.np_round_to(rng.standard_normal((C1, 1, 3, 3)).astype(np.float32) * 0.3, dtype)
    # (W2 small enough that the sums over up to 512 intermediate channels stay below 2: one bf16 step there is
    # 2^-7, inside the absolute bound)
    W2 = oracle.np_round_to(rng.standard_normal((C2, C1, 1, 1)).astype(np.float32) * 0.02, dtype)
    x, w1, w2 = to_dev(X, dtype), to_dev(W1, dtype), to_dev(W2, dtype)
    for relu in (False, True):
        y = torch.full((N, C2, H, W), float("nan"), device=x.device, dtype=x.dtype)
        desc = chain.conv_chain_desc(x, w1, w2, y, 1, 1, 0, 1, "relu" if relu else "cast", relu, C0)
        assert chain.select_tile(desc).variant == 4025
        chain.run_conv_chain(x, w1, w2, y, desc=desc)
        torch.cuda.synchronize()
        got = y.float().cpu().numpy()
        assert np.isfinite(got).all()
        want = oracle.conv_chain_f32(X, W1, W2, 1, 1, 0, 1, relu_mid=relu, relu_out=relu, round_mid=dtype, groups1=C0)
        mx, rel = errors(got, oracle.np_round_to(want, dtype))
        if dtype == "bfloat16" and relu:
            report("conv chain (wide second filter / depthwise) bf16 rows x16 %s" % (case,), mx, rel)
        assert mx <= MAX_ABS and rel <= REL_L2, (relu, mx, rel)
        y2 = torch.full_like(y, float("nan"))
        desc2 = chain.conv_chain_desc(x, w1, w2, y2, 1, 1, 0, 1, "relu" if relu else "cast", relu, C0, tile_variant=4000)
        assert chain.select_tile(desc2).variant % 10 == 2
        chain.run_conv_chain(x, w1, w2, y2, desc=desc2)
        torch.cuda.synchronize()
        assert torch.equal(y, y2), (relu, errors(got, y2.float().cpu().numpy()))


def test_row_streaming_kernel_steps_aside_for_less_aligned_pointers(oracle):
    """x or y not 16-byte aligned: the call runs on the persistent kernel instead (same result within tolerance)."""
    N, C0, H, W, C2 = 1, 16, 16, 24, 32
    rng = np.random.default_rng(3)
    X = oracle.np_round_to(rng.standard_normal((N, C0, H, W)).astype(np.float32), "float16")
    W1 = oracle.np_round_to(rng.standard_normal((C0, 1, 3, 3)).astype(np.float32) * 0.3, "float16")
    W2 = oracle.np_round_to(rng.standard_normal((C2, C0, 1, 1)).astype(np.float32) * 0.2, "float16")
    x, w1, w2 = to_dev(X, "float16"), to_dev(W1, "float16"), to_dev(W2, "float16")
    want = oracle.np_round_to(oracle.conv_chain_f32(X, W1, W2, 1, 1, 0, 1, round_mid="float16", groups1=C0), "float16")
    xbuf = torch.zeros(x.numel() + 8, device=x.device, dtype=torch.float16)
    ybuf = torch.zeros(N * C2 * H * W + 8, device=x.device, dtype=torch.float16)
    for xo, yo in ((0, 0), (4, 0), (0, 4), (1, 2)):
        xs = xbuf[xo:xo + x.numel()].view_as(x)
        xs.copy_(x)
        ys = ybuf[yo:yo + N * C2 * H * W].view(N, C2, H, W)
        ys.fill_(float("nan"))
        chain.run_conv_chain(xs, w1, w2, ys, groups1=C0)
        torch.cuda.synchronize()
        mx, rel = errors(ys.float().cpu().numpy(), want)
        assert mx <= MAX_ABS and rel <= REL_L2, (xo, yo, mx, rel)


def test_depthwise_chain_with_less_aligned_pointers(oracle):
    """x only 2-byte aligned (narrower halo loads) and y only 4-byte aligned (2-byte stores instead
    of the 16-byte path) must give the same bits as the aligned call."""
    N, C0, H, W, factor, C2 = 1, 8, 16, 16, 16, 64
    C1 = C0 * factor
    rng = np.random.default_rng(11)
    X = oracle.np_round_to(rng.standard_normal((N, C0, H, W)).astype(np.float32), "float16")
    W1 = oracle.np_round_to(rng.standard_normal((C1, 1, 3, 3)).astype(np.float32) * 0.3, "float16")
    W2 = oracle.np_round_to(rng.standard_normal((C2, C1, 1, 1)).astype(np.float32) * 0.05, "float16")
    x, w1, w2 = to_dev(X, "float16"), to_dev(W1, "float16"), to_dev(W2, "float16")
    want = torch.empty(N, C2, H, W, device=x.device, dtype=torch.float16)
    chain.run_conv_chain(x, w1, w2, want, groups1=C0)
    xbuf = torch.zeros(x.numel() + 8, device=x.device, dtype=torch.float16)
    ybuf = torch.zeros(want.numel() + 8, device=x.device, dtype=torch.float16)
    for xo, yo in ((1, 0), (0, 2), (3, 6), (4, 0)):  # the last: x 8-byte aligned, 4-element halo vectors
        xs = xbuf[xo:xo + x.numel()].view_as(x)
        xs.copy_(x)
        ys = ybuf[yo:yo + want.numel()].view_as(want)
        ys.fill_(float("nan"))
        chain.run_conv_chain(xs, w1, w2, ys, groups1=C0)
        torch.cuda.synchronize()
        assert torch.equal(ys, want), (xo, yo)
    mx, rel = errors(want.float().cpu().numpy(),
                     oracle.conv_chain_f32(X, W1, W2, 1, 1, 0, 1, round_mid="float16", groups1=C0))
    assert mx <= MAX_ABS and rel <= REL_L2


def test_depthwise_chain_rejects():
    x = torch.zeros(1, 16, 14, 14, device="cuda:0", dtype=torch.float16)
    y = torch.zeros(1, 32, 14, 14, device="cuda:0", dtype=torch.float16)
    with pytest.raises(NotImplementedError):  # factor 3
        chain.run_conv_chain(x, torch.zeros(48, 1, 3, 3, device="cuda:0", dtype=torch.float16),
                             torch.zeros(32, 48, 1, 1, device="cuda:0", dtype=torch.float16), y, groups1=16)
    with pytest.raises(NotImplementedError):  # 5x5 depthwise filter
        chain.run_conv_chain(x, torch.zeros(16, 1, 5, 5, device="cuda:0", dtype=torch.float16),
                             torch.zeros(32, 16, 1, 1, device="cuda:0", dtype=torch.float16), y, 2, groups1=16)
    with pytest.raises(ValueError):  # groups that are neither 1 nor C0
        chain.run_conv_chain(x, torch.zeros(16, 4, 3, 3, device="cuda:0", dtype=torch.float16),
                             torch.zeros(32, 16, 1, 1, device="cuda:0", dtype=torch.float16), y, groups1=4)


def test_conv_chain_rejects_what_it_cannot_fuse():
    x = torch.zeros(1, 16, 14, 14, device="cuda:0", dtype=torch.float16)
    w1 = torch.zeros(32, 16, 1, 1, device="cuda:0", dtype=torch.float16)
    with pytest.raises(NotImplementedError):  # 5x5 second filter
        chain.run_conv_chain(x, w1, torch.zeros(32, 32, 5, 5, device="cuda:0", dtype=torch.float16),
                             torch.zeros(1, 32, 14, 14, device="cuda:0", dtype=torch.float16), 0, 1, 2, 1)
    with pytest.raises(NotImplementedError):  # second convolution with a stride beyond 4
        chain.run_conv_chain(x, w1, torch.zeros(32, 32, 3, 3, device="cuda:0", dtype=torch.float16),
                             torch.zeros(1, 32, 3, 3, device="cuda:0", dtype=torch.float16), 0, 1, 1, 5)


CASES_STRIDED_SECOND = [
    # N, C0, H, W, C1, R1, pad1, stride1, C2, R2, pad2, stride2, groups1
    (2, 32, 30, 30, 64, 3, 1, 1, 64, 1, 0, 2, 1),     # 3x3 -> 1x1 keeping every second pixel
    (1, 24, 29, 31, 40, 3, 1, 2, 48, 1, 0, 2, 1),     # both strided, odd extents
    (1, 64, 56, 56, 64, 1, 0, 1, 128, 1, 0, 2, 1),    # 1x1 -> 1x1 stride 2 (a ResNet downsampling branch)
    (2, 16, 28, 28, 16, 3, 1, 1, 32, 1, 0, 2, 16),    # depthwise first convolution
    (1, 32, 29, 29, 64, 1, 0, 1, 64, 3, 1, 2, 1),     # 1x1 -> 3x3 stride 2
    (2, 16, 20, 36, 32, 3, 1, 1, 40, 3, 0, 2, 1),     # 3x3 -> 3x3 stride 2 without padding
    (1, 16, 33, 17, 24, 3, 1, 1, 32, 3, 1, 3, 1),     # stride 3
    (1, 32, 14, 14, 192, 1, 0, 1, 64, 3, 1, 1, 1),    # 192 intermediate channels under a 3x3 second filter
    (2, 64, 20, 24, 256, 1, 0, 1, 96, 3, 1, 1, 1),    # 256
    (1, 32, 15, 15, 256, 1, 0, 1, 32, 3, 1, 2, 1),    # 256, strided
]


@pytest.mark.parametrize("case", CASES_STRIDED_SECOND)
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_strided_second_convolution_and_wide_intermediates(oracle, case, dtype):
    """Second convolutions with a stride (a strided 1x1 is run as the chain whose first convolution carries both
    strides; a strided 3x3 reads the intermediate tile in LDS with that stride) and 3x3 second convolutions over up
    to 256 intermediate channels."""
    N, C0, H, W, C1, R1, pad1, stride1, C2, R2, pad2, stride2, groups1 = case
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, R1, R2, dtype, seed=C0 + C2 + stride2, w_std=0.05)
    if groups1 != 1:  # depthwise: one filter per channel
        W1 = oracle.np_round_to(np.random.default_rng(C0).standard_normal((C1, 1, R1, R1)).astype(np.float32) * 0.3, dtype)
    for relu in (False, True):
        want32 = oracle.conv_chain_f32(X, W1, W2, pad1, stride1, pad2, stride2, relu_mid=relu, relu_out=relu,
                                       round_mid=dtype, groups1=groups1)
        got32 = run_conv(X, W1, W2, dtype, pad1, stride1, "relu" if relu else "cast", relu, "float32", None, pad2,
                         groups1, 0, stride2)
        assert got32.shape == want32.shape and np.isfinite(got32).all()
        mx, rel = errors(got32, want32)
        assert mx <= MAX_ABS and rel <= REL_L2, (relu, mx, rel)
    got = run_conv(X, W1, W2, dtype, pad1, stride1, "relu", True, None, None, pad2, groups1, 0, stride2)
    mx, rel = errors(got, oracle.np_round_to(want32, dtype))
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)


def test_conv_relu_conv_relu_vs_torch(oracle):
    # the reference's GPU check: conv3x3 -> ReLU -> conv -> ReLU vs torch conv2d, uniform(-1,1)
    # inputs, rtol = atol = 0.1 (testing/hyper_fusion/conv_relu_conv_relu_fuse_hw_cuda.py:750-793);
    # here with a 1x1 second convolution and the workload tolerance
    rng = np.random.default_rng(4)
    N, C0, H, W, C1, C2 = 2, 32, 16, 16, 64, 64
    X = oracle.np_round_to(rng.uniform(-1, 1, (N, C0, H, W)).astype(np.float32), "float16")
    W1 = oracle.np_round_to(rng.uniform(-1, 1, (C1, C0, 3, 3)).astype(np.float32) * 0.1, "float16")
    W2 = oracle.np_round_to(rng.uniform(-1, 1, (C2, C1, 1, 1)).astype(np.float32) * 0.1, "float16")
    got = run_conv(X, W1, W2, "float16", inter="relu", relu_out=True, out_dtype="float32")
    t = torch.nn.functional
    mid = t.conv2d(torch.from_numpy(X).double(), torch.from_numpy(W1).double(), padding=1).clamp_min(0)
    mid = mid.float().half().double()
    want = t.conv2d(mid, torch.from_numpy(W2).double()).clamp_min(0).numpy()
    assert (got >= 0).all()
    assert np.allclose(got, want, rtol=0.1, atol=0.1)
    mx, rel = errors(got, want)
    assert mx <= MAX_ABS and rel <= REL_L2
    want_o = oracle.conv_chain_f32(X, W1, W2, relu_mid=True, relu_out=True, round_mid="float16")
    assert errors(got, want_o)[1] <= REL_L2


def test_conv_chain_delta_filter(oracle):
    # a 3x3 filter with a single one shifts the image; the 1x1 then mixes channels exactly
    rng = np.random.default_rng(6)
    X = oracle.np_round_to(rng.integers(-4, 5, (1, 16, 10, 12)).astype(np.float32), "float16")
    W1 = np.zeros((16, 16, 3, 3), np.float32)
    for c in range(16):
        W1[c, c, 2, 0] = 1.0  # y[p][q] = x[p+1][q-1]
    W2 = rng.integers(-2, 3, (8, 16, 1, 1)).astype(np.float32)
    got = run_conv(X, W1, W2, "float16", out_dtype="float32")
    shifted = np.zeros_like(X)
    shifted[:, :, :-1, 1:] = X[:, :, 1:, :-1]
    want = np.einsum("kc,nchw->nkhw", W2[:, :, 0, 0], shifted)
    assert np.array_equal(got, want)  # small integers: exact


def test_conv_chain_full_size_linearity(oracle):
    # the full configuration (N=32, 64 -> 64 3x3 on 56x56, then 64 -> 256): checked against the
    # checker on two images and through linearity in W2 on all of them
    N, C0, H, W, C1, C2 = 32, 64, 56, 56, 64, 256
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, 3, 1, "float16", seed=0)
    got = run_conv(X, W1, W2, "float16", out_dtype="float32")
    sel = [0, 31]
    want = oracle.conv_chain_f32(X[sel], W1, W2, round_mid="float16")
    mx, rel = errors(got[sel], want)
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)
    W2a = oracle.np_round_to(W2 * 0.5, "float16")
    W2b = W2 - W2a
    assert np.array_equal(oracle.np_round_to(W2b, "float16"), W2b)
    s = run_conv(X, W1, W2a, "float16", out_dtype="float32") + run_conv(X, W1, W2b, "float16", out_dtype="float32")
    assert errors(s, got)[1] <= 1e-5


def test_row_pipeline_conv3x3_conv1x1_at_benchmark_size(oracle):
    """The benchmarked kernel of the conv3x3 -> conv1x1 configuration at its size (N = 32, fp16 output, variant 3707:
    bands of 7 rows, one workgroup per compute unit): three images against the checker, all of them against the
    general kernel on the same inputs, and linearity in W2 over all of them."""
    N, C0, H, W, C1, C2 = 32, 64, 56, 56, 64, 256
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, 3, 1, "float16", seed=0)
    x, w1, w2 = to_dev(X, "float16"), to_dev(W1, "float16"), to_dev(W2, "float16")
    y = torch.full((N, C2, H, W), float("nan"), device=x.device, dtype=torch.float16)
    desc = chain.conv_chain_desc(x, w1, w2, y, 1, 1, 0, 1, "cast", False)
    assert chain.select_tile(desc).variant == 3707
    chain.run_conv_chain(x, w1, w2, y, desc=desc)
    torch.cuda.synchronize()
    got = y.float().cpu().numpy()
    assert np.isfinite(got).all()
    for n in (0, 13, 31):
        want = oracle.conv_chain_f32(X[n:n + 1], W1, W2, round_mid="float16")
        mx, rel = errors(got[n:n + 1], oracle.np_round_to(want, "float16"))
        assert mx <= MAX_ABS and rel <= REL_L2, (n, mx, rel)
    y2 = torch.full_like(y, float("nan"))
    desc2 = chain.conv_chain_desc(x, w1, w2, y2, 1, 1, 0, 1, "cast", False, tile_variant=3000)
    assert chain.select_tile(desc2).variant == 3022
    chain.run_conv_chain(x, w1, w2, y2, desc=desc2)
    torch.cuda.synchronize()
    mx, rel = errors(got, y2.float().cpu().numpy())  # two summation orders, both rounded to fp16 at the end
    assert mx <= MAX_ABS and rel <= 5e-4, (mx, rel)
    # W2 = W2a + W2b with both parts exact in fp16: the two outputs add up to the whole one but for their roundings
    W2a = oracle.np_round_to(W2 * 0.5, "float16")
    W2b = W2 - W2a
    assert np.array_equal(oracle.np_round_to(W2b, "float16"), W2b)
    ya, yb = torch.empty_like(y), torch.empty_like(y)
    chain.run_conv_chain(x, w1, to_dev(W2a, "float16"), ya, desc=desc)
    chain.run_conv_chain(x, w1, to_dev(W2b, "float16"), yb, desc=desc)
    torch.cuda.synchronize()
    mx, rel = errors(ya.float().cpu().numpy() + yb.float().cpu().numpy(), got)
    assert rel <= 5e-4, (mx, rel)  # three fp16 roundings of O(1) values: 2^-11 / sqrt(3) each


@pytest.mark.parametrize("mult,variant", [(1, 4024), (16, 4025)])
def test_row_streaming_depthwise_chains_at_benchmark_size(oracle, mult, variant):
    """The two depthwise workloads of the benchmark at their size (32 x 32 x 112 x 112 -> 64, multiplier 1 and 16):
    the benchmarked row-streaming kernel on three images against the checker, on all of them against the tile kernel
    (tile_variant 4000), and linear in x (a power of two only shifts exponents)."""
    N, C0, H, W, C2 = 32, 32, 112, 112, 64
    C1 = C0 * mult
    rng = np.random.default_rng(40 + mult)
    X = oracle.np_round_to(rng.standard_normal((N, C0, H, W)).astype(np.float32), "float16")
    W1 = oracle.np_round_to(rng.standard_normal((C1, 1, 3, 3)).astype(np.float32) * 0.3, "float16")
    W2 = oracle.np_round_to(rng.standard_normal((C2, C1, 1, 1)).astype(np.float32) * (0.2 if mult == 1 else 0.05), "float16")
    x, w1, w2 = to_dev(X, "float16"), to_dev(W1, "float16"), to_dev(W2, "float16")
    y = torch.full((N, C2, H, W), float("nan"), device=x.device, dtype=torch.float16)
    desc = chain.conv_chain_desc(x, w1, w2, y, 1, 1, 0, 1, "relu", False, C0)
    assert chain.select_tile(desc).variant == variant
    chain.run_conv_chain(x, w1, w2, y, desc=desc)
    torch.cuda.synchronize()
    got = y.float().cpu().numpy()
    assert np.isfinite(got).all()
    for n in (0, 18, 31):
        want = oracle.conv_chain_f32(X[n:n + 1], W1, W2, 1, 1, 0, 1, relu_mid=True, round_mid="float16", groups1=C0)
        mx, rel = errors(got[n:n + 1], oracle.np_round_to(want, "float16"))
        assert mx <= MAX_ABS and rel <= REL_L2, (n, mx, rel)
    y2 = torch.full_like(y, float("nan"))
    desc2 = chain.conv_chain_desc(x, w1, w2, y2, 1, 1, 0, 1, "relu", False, C0, tile_variant=4000)
    assert chain.select_tile(desc2).variant not in (4024, 4025)
    chain.run_conv_chain(x, w1, w2, y2, desc=desc2)
    torch.cuda.synchronize()
    mx, rel = errors(got, y2.float().cpu().numpy())
    assert mx <= MAX_ABS and rel <= 5e-4, (mx, rel)
    ya, yb = torch.empty_like(y), torch.empty_like(y)
    chain.run_conv_chain(x, w1, w2, ya, 1, 1, 0, 1, "cast", False, groups1=C0)
    chain.run_conv_chain(x * 2, w1, w2, yb, 1, 1, 0, 1, "cast", False, groups1=C0)
    torch.cuda.synchronize()
    mx, rel = errors((ya * 2).float().cpu().numpy(), yb.float().cpu().numpy())
    assert mx <= 1e-3 and rel <= 1e-5, (mx, rel)


@pytest.mark.skip(reason=PERSIST_OFF)
def test_persistent_conv_chain_full_size(oracle):
    # the full configuration through the opt-in persistent kernel: two images against the checker, all
    # of them against the default kernel (two summation orders, both rounded to fp16 at the end)
    N, C0, H, W, C1, C2 = 32, 64, 56, 56, 64, 256
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, 3, 1, "float16", seed=1)
    default = run_conv(X, W1, W2, "float16", inter="relu", relu_out=True)
    got = run_conv(X, W1, W2, "float16", inter="relu", relu_out=True, tile_variant=3900)
    sel = [0, 31]
    want = oracle.np_round_to(oracle.conv_chain_f32(X[sel], W1, W2, relu_mid=True, relu_out=True, round_mid="float16"),
                              "float16")
    mx, rel = errors(got[sel], want)
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)
    assert np.isfinite(got).all() and errors(got, default)[1] <= REL_L2
    assert (got >= 0).all() and (got == 0).mean() > 0.2  # the output ReLU took effect


def test_conv_chain_rejects_unsupported():
    dev = "cuda:0"
    x = torch.zeros(1, 16, 8, 8, device=dev, dtype=torch.float16)
    w1 = torch.zeros(16, 16, 3, 3, device=dev, dtype=torch.float16)
    w2 = torch.zeros(16, 16, 3, 3, device=dev, dtype=torch.float16)
    y = torch.zeros(1, 16, 8, 8, device=dev, dtype=torch.float16)
    with pytest.raises(ValueError):
        chain.run_conv_chain(x, w1, w2[:, :, :1, :1].contiguous(), y[:, :8].contiguous(), 1, 1, 0, 1)


@pytest.mark.parametrize("case", [CASES[0], CASES[2], CASES_3X3_SECOND[0], CASES_3X3_SECOND[3]])
def test_prepared_weights_give_the_same_bits(oracle, case):
    """ditto_conv_chain_prepare + ditto_conv_chain_run_prepared == ditto_conv_chain_run."""
    if len(case) == 9:
        N, C0, H, W, C1, R1, pad1, stride1, C2 = case
        R2, pad2 = 1, 0
    else:
        N, C0, H, W, C1, R1, pad1, stride1, C2, R2, pad2 = case
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, R1, R2, "float16", seed=3, w_std=0.05)
    x, w1, w2 = to_dev(X, "float16"), to_dev(W1, "float16"), to_dev(W2, "float16")
    P = (H + 2 * pad1 - R1) // stride1 + 1 + 2 * pad2 - R2 + 1
    Q = (W + 2 * pad1 - R1) // stride1 + 1 + 2 * pad2 - R2 + 1
    want = torch.full((N, C2, P, Q), float("nan"), device=x.device, dtype=torch.float16)
    got = want.clone()
    desc = chain.conv_chain_desc(x, w1, w2, want, pad1, stride1, pad2, 1, "relu", True)
    chain.run_conv_chain(x, w1, w2, want, desc=desc)
    ws = chain.prepare_conv_chain(desc, w1, w2)
    assert ws.numel() >= chain.conv_chain_workspace_bytes(desc) > 0
    for _ in range(2):  # the workspace is read-only for the prepared call
        got.fill_(float("nan"))
        chain.run_conv_chain(x, w1, w2, got, desc=desc, workspace=ws, prepared=True)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
    with pytest.raises(ValueError):  # no workspace, nothing prepared
        chain.run_conv_chain(x, w1, w2, got, desc=desc, prepared=True)
    small = torch.empty(16, dtype=torch.uint8, device=x.device)
    with pytest.raises(ValueError):
        chain.prepare_conv_chain(desc, w1, w2, workspace=small)


def test_conv_tile_variant_tuning_round_trip(tmp_path, oracle):
    """The measurement-driven kernel choice for conv chains: every family that can run the shape is timed with
    prepared weights, logged in the reference's JSON-lines format (chimera_integrate.py:326-333, 527-556), and
    the logged winner is what a later call is steered to."""
    from ditto_amd.auto_schedule.schedulers import chimera_integrate as ci

    N, C0, H, W, C1, C2 = 4, 64, 56, 56, 64, 256
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, 3, 1, "float16", seed=9)
    x, w1, w2 = to_dev(X, "float16"), to_dev(W1, "float16"), to_dev(W2, "float16")
    y = torch.full((N, C2, H, W), float("nan"), device=x.device, dtype=torch.float16)
    desc = chain.conv_chain_desc(x, w1, w2, y)
    space = ci.make_conv_tile_variant_space(desc)
    assert sorted(t["variant"] // 100 for t in space) == [30, 37]
    log = str(tmp_path / "chimera_conv.log")
    key = ci.conv_workload_key(desc)
    best = ci.select_conv_tile_variant(key, log, x, w1, w2, y, min_repeat_ms=5)
    assert len(open(log).read().strip().splitlines()) == len(space)
    assert ci.load_best_records(log)[key]["record"]["variant"] == best.record["variant"] and 0 < best.value < 5.0
    assert ci.auto_schedule_conv_chain_hip(key, log, x, w1, w2, y) == best.record["variant"]
    chain.run_conv_chain(x, w1, w2, y, tile_variant=best.record["variant"])
    torch.cuda.synchronize()
    want = oracle.conv_chain_f32(X[:1], W1, W2, round_mid="float16")
    mx, rel = errors(y[:1].float().cpu().numpy(), oracle.np_round_to(want, "float16"))
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)


def test_overflowed_outputs_of_the_conv1x1_conv3x3_row_pipeline():
    """An fp16 output that overflows: the kernels that keep W2 in LDS (tile_variant 3600) and the general one (3500)
    confine the infinity to its own channel, as the reference's chain does.  The row pipeline (38xx, the default
    for this shape) passes the cast result through an identity MFMA on its way to the 8-pixel stores, where
    0 x inf is NaN: the overflowed value itself comes out infinite, the other channels of the same pixel within
    its block of 32 come out NaN instead of their finite values, and every other pixel is untouched.  A caller
    that needs the exact semantics on overflowing data asks for tile_variant 3600."""
    N, C0, H, W, C1, C2 = 1, 64, 16, 16, 64, 64
    dev = "cuda:0"
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(N, C0, H, W, generator=g) * 4).half().to(dev)
    w1 = (torch.randn(C1, C0, 1, 1, generator=g) * 0.05).half().to(dev)
    w2 = (torch.randn(C2, C1, 3, 3, generator=g) * 0.05).half().to(dev)
    w2[5] *= 20000.0     # channel 5 of the output (standard deviation about 4e4) overflows fp16 at some pixels
    outs = {}
    for tv in (0, 3600, 3500):
        y = torch.full((N, C2, H, W), float("nan"), device=dev, dtype=torch.float16)
        desc = chain.conv_chain_desc(x, w1, w2, y, 0, 1, 1, 1, "cast", False, tile_variant=tv)
        if tv == 0:
            assert chain.select_tile(desc).variant // 100 == 38
        chain.run_conv_chain(x, w1, w2, y, desc=desc)
        torch.cuda.synchronize()
        outs[tv] = y.float().cpu()
    ref = torch.nn.functional.conv2d(torch.nn.functional.conv2d(x.float(), w1.float()).half().float(), w2.float(),
                                     padding=1).half().float().cpu()
    over = torch.isinf(ref[0, 5])
    assert over.any() and not over.all() and not torch.isinf(ref[0, :5]).any() and not torch.isinf(ref[0, 6:]).any()
    for tv in (3600, 3500):  # exact semantics: infinities where the reference has them, everything else finite and close
        o = outs[tv]
        assert torch.equal(torch.isinf(o), torch.isinf(ref)) and not torch.isnan(o).any(), tv
        fin = ~torch.isinf(ref)
        assert bool(((o[fin] - ref[fin]).abs() <= 2e-3 * ref[fin].abs() + 1e-2).all()), tv
    o = outs[0]
    assert torch.equal(torch.isinf(o[0, 5]), over)                      # the overflowed values themselves
    clean = ~over                                                        # pixels without an overflow: untouched
    assert not torch.isnan(o[0][:, clean]).any()
    assert float((o[0, :5][:, clean] - ref[0, :5][:, clean]).abs().max()) <= 1e-2
    assert not torch.isnan(o[0, 32:]).any()                              # the other block of 32 channels: untouched
    assert torch.isnan(o[0, :32][:, over]).sum() > 0                     # the documented divergence


@pytest.mark.parametrize("first", ["3x3", "1x1"])
def test_packed_placeholders_of_the_reference(oracle, first):
    """The reference's calling convention for its GPU conv drivers: packed, pre-padded tensors
    (conv3x3_conv1x1_cuda.py:90-105 and :164-170; conv1x1_conv3x3_cuda.py:90-105).  The built function takes them as they
    are; the index maps are restated here with plain loops-free numpy against the NCHW result of the checker,
    including a border the caller filled with something other than zeros (which the reference's index expression
    reads like any other pixel)."""
    import ditto_amd as ditto
    from ditto_amd import auto_compute as ac, layout
    from ditto_amd.drivers import common

    N, C0, H, W, C1, C2 = 2, 32, 12, 16, 64, 48
    Fn = ac.nn.functional
    if first == "3x3":
        ins, outs = Fn.Conv3x3Conv1x1(N, C0, H, W, C1, C2)
        R1, R2, pad1, pad2 = 3, 1, 1, 0
    else:
        ins, outs = Fn.Conv1x1Conv3x3(N, C0, H, W, C1, C2)
        R1, R2, pad1, pad2 = 1, 3, 0, 1
    layer = ac.layer([outs[0].op], inputs=[ins[0]], weights=ins[1:])
    func = ditto.build(common.describe_layer(layer), layer.schedule_tensors, "hip")
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, R1, R2, "float16", seed=31, w_std=0.05)
    rng = np.random.default_rng(2)
    # the packed image as the reference's host code lays it out: [N, C/16, H + 2 pad, W + 2 pad + 1, 16], border NOT zero
    Xp = rng.standard_normal((N, C0, H + 2 * pad1, W + 2 * pad1)).astype(np.float32)
    Xp = oracle.np_round_to(Xp, "float16")
    Xp[:, :, pad1:pad1 + H, pad1:pad1 + W] = X
    img_np = np.zeros((N, C0 // 16, H + 2 * pad1, W + 2 * pad1 + 1, 16), np.float32)
    img_np[:, :, :, :W + 2 * pad1, :] = Xp.reshape(N, C0 // 16, 16, H + 2 * pad1, W + 2 * pad1).transpose(0, 1, 3, 4, 2)
    w1_np = W1.reshape(C1 // 16, 16, C0 // 16, 16, R1, R1).transpose(4, 5, 2, 0, 3, 1)      # [r, s, co, ko, ci, ki]
    w2_np = W2.reshape(C2 // 16, 16, C1 // 16, 16, R2, R2).transpose(4, 5, 2, 0, 3, 1)
    if R1 == 1:
        w1_np = w1_np[0, 0]
    if R2 == 1:
        w2_np = w2_np[0, 0]
    img_p, w1_p, w2_p = (to_dev(np.ascontiguousarray(t), "float16") for t in (img_np, w1_np, w2_np))
    out_p = torch.full((N, C2 // 16, H, W, 16), float("nan"), device=img_p.device, dtype=torch.float16)
    func(img_p, w1_p, w2_p, out_p)
    torch.cuda.synchronize()
    # the checker on the padded image without further padding of the first convolution
    want = oracle.conv_chain_f32(Xp, W1, W2, 0, 1, pad2, 1, round_mid="float16")
    got = out_p.float().cpu().numpy().transpose(0, 1, 4, 2, 3).reshape(N, C2, H, W)
    mx, rel = errors(got, oracle.np_round_to(want, "float16"))
    assert mx <= MAX_ABS and rel <= REL_L2, (mx, rel)
    # the layout helpers are each other's inverses, and agree with the maps written out above
    assert torch.equal(layout.pack_weight(layout.unpack_weight(w1_p)), w1_p)
    assert torch.equal(layout.unpack_image(img_p, W + 2 * pad1).float().cpu(), torch.from_numpy(Xp))
    assert torch.equal(layout.pack_image(to_dev(X, "float16"), pad1, 1)[:, :, pad1:pad1 + H, pad1:pad1 + W],
                       img_p[:, :, pad1:pad1 + H, pad1:pad1 + W])
    # a second call with the same packed weights reuses their unpacked form; updated weights are unpacked again
    cached = func._packed_weights[3]
    func(img_p, w1_p, w2_p, out_p)
    assert func._packed_weights[3] is cached
    w1_p.mul_(0.5)
    func(img_p, w1_p, w2_p, out_p)
    torch.cuda.synchronize()
    got2 = out_p.float().cpu().numpy().transpose(0, 1, 4, 2, 3).reshape(N, C2, H, W)
    want2 = oracle.conv_chain_f32(Xp, W1 * 0.5, W2, 0, 1, pad2, 1, round_mid="float16")
    assert errors(got2, oracle.np_round_to(want2, "float16"))[1] <= REL_L2
