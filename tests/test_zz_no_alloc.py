"""``ditto_conv_chain_run_static``: the conv chain entry point that allocates nothing (its workspace is a
device array inside the library) against ``ditto_conv_chain_run`` with a caller workspace.  Same kernels,
so the outputs are compared bit for bit; two calls in a row share the array, the second with a smaller
input."""
import ctypes

import numpy as np
import pytest
import torch

from ditto_amd import _lib, chain
from tests.gpu_util import to_dev, TORCH_DTYPES

pytestmark = pytest.mark.gpu


def _both(oracle, case, dtype, seed):
    N, C0, H, W, C1, R1, pad1, C2, R2, pad2 = case
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, R1, R2, dtype, seed=seed, w_std=0.05)
    x, w1, w2 = to_dev(X, dtype), to_dev(W1, dtype), to_dev(W2, dtype)
    P = H + 2 * pad1 - R1 + 1 + 2 * pad2 - R2 + 1
    Q = W + 2 * pad1 - R1 + 1 + 2 * pad2 - R2 + 1
    want = torch.full((N, C2, P, Q), float("nan"), device=x.device, dtype=TORCH_DTYPES[dtype])
    got = torch.full_like(want, float("nan"))
    desc = chain.conv_chain_desc(x, w1, w2, want, pad1, 1, pad2, 1, "relu", True)
    nbytes = chain.conv_chain_workspace_bytes(desc)
    assert 0 < nbytes <= _lib.STATIC_WORKSPACE_BYTES
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    chain.run_conv_chain(x, w1, w2, want, desc=desc, workspace=ws)
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    print("static conv chain", case, dtype, flush=True)
    _lib.check(lib.ditto_conv_chain_run_static(ctypes.byref(desc), x.data_ptr(), w1.data_ptr(), w2.data_ptr(),
                                               got.data_ptr(), stream))
    torch.cuda.synchronize()
    return got.float().cpu().numpy(), want.float().cpu().numpy()


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_static_workspace_entry_matches_the_workspace_entry(oracle, dtype):
    # N, C0, H, W, C1, R1, pad1, C2, R2, pad2: first the larger weights, then a smaller chain into the same array
    for seed, case in enumerate([(4, 64, 56, 56, 64, 3, 1, 256, 1, 0), (2, 16, 24, 24, 32, 3, 1, 48, 1, 0),
                                 (3, 64, 28, 32, 64, 1, 0, 64, 3, 1), (1, 8, 16, 16, 16, 1, 0, 16, 3, 1)]):
        got, want = _both(oracle, case, dtype, seed)
        assert np.isfinite(want).all() and np.abs(want).max() > 0
        assert np.array_equal(got, want), case


def test_static_workspace_entry_rejects_what_does_not_fit():
    dev = "cuda:0"
    # 256 x 1024 x 3 x 3 fp16 weights repack to more than the static array holds
    x = torch.zeros(1, 1024, 8, 8, device=dev, dtype=torch.float16)
    w1 = torch.zeros(256, 1024, 3, 3, device=dev, dtype=torch.float16)
    w2 = torch.zeros(32, 256, 1, 1, device=dev, dtype=torch.float16)
    y = torch.zeros(1, 32, 8, 8, device=dev, dtype=torch.float16)
    desc = chain.conv_chain_desc(x, w1, w2, y, 1, 1, 0, 1)
    assert chain.conv_chain_workspace_bytes(desc) > _lib.STATIC_WORKSPACE_BYTES
    rc = _lib.load().ditto_conv_chain_run_static(ctypes.byref(desc), x.data_ptr(), w1.data_ptr(), w2.data_ptr(),
                                                 y.data_ptr(), None)
    assert rc == _lib.EWORKSPACE and "static workspace" in _lib.last_error()


def test_static_workspace_entry_under_graph_capture(oracle):
    """The use the entry point is for: after one call outside any capture (which takes the array's address and
    configures the kernels on this device), the call is recorded into a HIP graph -- an allocation inside it would
    fail the capture -- and every replay gives the eager result."""
    case, dtype = (2, 64, 56, 56, 64, 3, 1, 256, 1, 0), "float16"
    N, C0, H, W, C1, R1, pad1, C2, R2, pad2 = case
    X, W1, W2 = oracle.make_conv_chain_inputs(N, C0, H, W, C1, C2, R1, R2, dtype, seed=21, w_std=0.05)
    x, w1, w2 = to_dev(X, dtype), to_dev(W1, dtype), to_dev(W2, dtype)
    y = torch.full((N, C2, H, W), float("nan"), device=x.device, dtype=TORCH_DTYPES[dtype])
    desc = chain.conv_chain_desc(x, w1, w2, y, pad1, 1, pad2, 1, "relu", True)
    lib = _lib.load()

    def call():
        stream = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.ditto_conv_chain_run_static(ctypes.byref(desc), x.data_ptr(), w1.data_ptr(), w2.data_ptr(),
                                                   y.data_ptr(), stream))

    call()  # the first call on the device: outside the capture
    torch.cuda.synchronize()
    want = y.clone()
    assert torch.isfinite(want).all()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call()
    for it in range(3):  # replays with eager work and synchronisations in between
        y.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), it
        call()
        torch.cuda.synchronize()
