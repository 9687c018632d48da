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


def test_attention_blocks_through_task_binding_and_graph_engine(tmp_path, oracle):
    """The flow of benchmark/chimera/cuda/bert_inference.py:59-129 for the attention layers: extract
    tasks, bind to the chimera scheduler, tune (log written), build, run through the graph engine;
    then ``test`` mode rebuilds from the log alone and must give the same numbers."""
    import json

    import numpy as np

    from ditto_amd.drivers import bert_inference

    kw = dict(dtype="float16", batch=2, seq_len=256, hidden=256, n_layers=3, attn_heads=4, number=5,
              log_dir=str(tmp_path))
    cost, outs, schedules = bert_inference.inference(test=False, **kw)
    assert 0 < cost < 50 and len(outs) == 3 and len(schedules) == 1
    logs = list(tmp_path.glob("chimera_*.log"))
    assert len(logs) == 1
    lines = [json.loads(l) for l in logs[0].read_text().splitlines()]
    assert lines and all(set(l) == {"wkl_key", "entry"} and l["entry"]["value"] > 0 for l in lines)
    (key,) = schedules
    best = min(lines, key=lambda l: l["entry"]["value"])["entry"]["record"]["variant"]
    assert schedules[key][0].tile_variant == best
    # test mode: nothing is measured, the schedule comes from the log
    before = logs[0].read_text()
    cost2, outs2, schedules2 = bert_inference.inference(test=True, hip_graph=False, **kw)
    assert logs[0].read_text() == before and schedules2[key][0].tile_variant == best

    # numbers: feed one known projection to every layer and compare with the CPU checker
    from ditto_amd import auto_schedule, chimera

    mha = ac.nn.module.MultiHeadAttentionMMA(4, 256, "float16", "float32", scale=None)
    graph = runtime.Graph([mha.layer(2, 256) for _ in range(2)], outputs=[(0, 0), (1, 0)])
    bound = chimera.task_binding(auto_schedule.extract_tasks_from_graph(graph))
    opt = auto_schedule.ScheduleOption("hip", log_file=str(tmp_path / logs[0].name[len("chimera_"):]))
    mods = {k: ditto.build(s, a, "hip") for k, (s, a) in auto_schedule.retrieve_schedule_bound_tasks(bound, opt).items()}
    rng = np.random.default_rng(7)
    qkv = oracle.np_round_to(rng.standard_normal((2, 256, 768)).astype(np.float32), "float16")
    x = torch.from_numpy(qkv).half().cuda()
    for make in (runtime.create_graph_engine, runtime.create_hip_graph_engine):
        eng = make(graph, mods, "cuda:0")
        eng.set_inputs([x, x])
        eng.compile()
        eng.run()
        torch.cuda.synchronize()
        q, k, v = (qkv[:, :, i * 256:(i + 1) * 256].reshape(2, 256, 4, 64).transpose(0, 2, 1, 3).reshape(8, 256, 64)
                   for i in range(3))
        want = oracle.bmm_chain_f64(q, np.ascontiguousarray(k.transpose(0, 2, 1)), v, inter="softmax", scale=0.125)
        want = want.reshape(2, 4, 256, 64).transpose(0, 2, 1, 3).reshape(2, 256, 256)
        for got in eng.get_outputs():
            err = np.abs(got.float().cpu().numpy() - want)
            assert err.max() <= 1e-2 and np.linalg.norm(err) / np.linalg.norm(want) <= 1e-3
