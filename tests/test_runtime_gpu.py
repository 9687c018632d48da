"""Graph engine over built chain layers (reference: src/runtime/graph_runtime.cc:14-260)."""
import pytest
import torch

import ditto_amd as ditto
from ditto_amd import auto_compute as ac
from ditto_amd import runtime
from ditto_amd.drivers import common

pytestmark = pytest.mark.gpu


def _two_layer_graph():
    batch, M, K, L, N = 4, 256, 64, 128, 64
    ins0, outs0 = ac.nn.functional.BatchGemmGemm(batch=batch, M=M, N=N, K=K, L=L, in_dtype="float16", acc_dtype="float32")
    l0, s0 = common.describe_bmm_chain(ins0, outs0, "float16", "float32", "gfx950")
    ins1, outs1 = ac.nn.functional.BatchGemmSoftmaxGemm(batch=batch, M=M, N=N, K=N, L=M, in_dtype="float16",
                                                        acc_dtype="float32", scale=0.125)
    l1, s1 = common.describe_bmm_chain(ins1, outs1, "float16", "float32", "gfx950")
    graph = runtime.Graph([l0, l1], edges={(1, 0): (0, 0)})
    mods = {l0.fingerprint: ditto.build(s0, l0.schedule_tensors, "hip"),
            l1.fingerprint: ditto.build(s1, l1.schedule_tensors, "hip")}
    return graph, mods


def _reference(a, b, c, key, value):
    mid = (a.float() @ b.float()).half().float() @ c.float()
    q = mid.half().float()
    return torch.softmax(q @ key.float() * 0.125, -1) @ value.float()


def test_graph_engine_runs_layers_in_order_and_times_them():
    graph, mods = _two_layer_graph()
    assert graph.graph_inputs == [(0, 0), (0, 1), (0, 2), (1, 1), (1, 2)]
    eng = runtime.create_graph_engine(graph, mods, "cuda:0")
    torch.manual_seed(0)
    dev = "cuda:0"
    a, b, c = (torch.randn(4, 256, 64, device=dev) * 0.25).half(), (torch.randn(4, 64, 128, device=dev) * 0.25).half(), \
        (torch.randn(4, 128, 64, device=dev) * 0.25).half()
    key, value = torch.randn(4, 64, 256, device=dev).half(), torch.randn(4, 256, 64, device=dev).half()
    eng.set_inputs([a, b, c, key, value])
    eng.compile()
    eng.run()
    torch.cuda.synchronize()
    (out,) = eng.get_outputs()
    ref = _reference(a, b, c, key, value)
    assert (out.float() - ref).abs().max().item() <= 2e-2
    ms = eng.timeit(20)
    assert 0 < ms < 5.0
    with pytest.raises(ValueError):
        eng.set_inputs([a, b, c])
    with pytest.raises(ValueError):
        runtime.Graph(graph.layers, edges={(1, 1): (0, 0)})  # shapes do not chain


def test_hip_graph_engine_replays_match_eager():
    graph, mods = _two_layer_graph()
    eager = runtime.create_graph_engine(graph, mods, "cuda:0")
    replay = runtime.create_cuda_graph_engine(graph, mods, "cuda:0")
    torch.manual_seed(1)
    dev = "cuda:0"
    ins = [(torch.randn(*graph.layers[li].inputs[ii].shape, device=dev) * 0.25).half() for li, ii in graph.graph_inputs]
    eager.set_inputs(ins)
    replay.set_inputs(ins)
    eager.run()
    torch.cuda.synchronize()
    want = eager.get_outputs()[0].clone()
    replay.compile()
    for it in range(4):  # replays with eager work and synchronisations in between
        replay.get_outputs()[0].zero_()
        torch.cuda.synchronize()
        replay.run()
        torch.cuda.synchronize()
        assert torch.equal(replay.get_outputs()[0], want), it
        eager.run()
        torch.cuda.synchronize()
    assert 0 < replay.timeit(20) < 5.0
