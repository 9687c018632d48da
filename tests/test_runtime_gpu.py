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


def test_graph_fusion_on_the_gpu(oracle):
    """A ReLU layer behind a GEMM chain and one behind a conv chain are folded into the chains by
    ``chimera.graph_fusion`` (reference: python/ditto/chimera/graph_fusion.py:4-52); the fused graph has one
    layer per chain and gives the numbers of chain-then-ReLU."""
    import numpy as np

    from ditto_amd import chimera, te
    from tests.gpu_util import errors, to_dev

    F = ac.nn.functional

    def relu_layer(shape, dtype="float16"):
        x = te.placeholder(shape, "x", dtype)
        return ac.layer([F.ReLU(x).op], inputs=[x], name="act")

    # GEMM chain -> ReLU -> GEMM chain
    batch, M, K, L, N = 2, 256, 64, 128, 64
    ins0, outs0 = F.BatchGemmGemm(batch, M, N, K, L, "float16", "float32")
    ins1, outs1 = F.BatchGemmGemm(batch, M, N, N, L, "float16", "float32", relu=True)
    l0 = ac.layer([outs0[0].op], inputs=ins0, name="chain0")
    l1 = ac.layer([outs1[0].op], inputs=ins1, name="chain1")
    graph = runtime.Graph([l0, relu_layer([batch, M, N]), l1], edges={(1, 0): (0, 0), (2, 0): (1, 0)})
    fused = chimera.graph_fusion(graph)
    assert len(fused.layers) == 2 and fused.layers[0].ops[0].kind == "relu_cast"
    mods = {l.fingerprint: ditto.build(common.describe_layer(l), l.schedule_tensors, "hip") for l in fused.layers}
    assert mods[fused.layers[0].fingerprint].sch.relu_out
    A, B, C = oracle.make_gemm_chain_inputs(batch, M, N, K, L, "float16", seed=3, std=0.25)
    _, B1, C1 = oracle.make_gemm_chain_inputs(batch, M, N, N, L, "float16", seed=4, std=0.25)
    for make in (runtime.create_graph_engine, runtime.create_hip_graph_engine):
        eng = make(fused, mods, "cuda:0")
        eng.set_inputs([to_dev(x, "float16") for x in (A, B, C, B1, C1)])
        eng.compile()
        eng.run()
        torch.cuda.synchronize()
        mid = oracle.np_round_to(np.maximum(oracle.bmm_chain_f64(A, B, C, inter="cast", round_mid="float16"), 0.0),
                                 "float16")
        want = oracle.bmm_chain_f64(mid, B1, C1, inter="relu", round_mid="float16")
        mx, rel = errors(eng.get_outputs()[0].float().cpu().numpy(), want)
        assert mx <= 1e-2 and rel <= 2e-3, (mx, rel)  # two chains deep: one rounding flip of the first moves the second

    # conv chain -> ReLU, weights as layer weights (the engine repacks them once per compile)
    n, c0, hw_, c1, c2 = 4, 32, 28, 64, 96
    cins, couts = F.Conv3x3Conv1x1(n, c0, hw_, hw_, c1, c2)
    cl = ac.layer([couts[0].op], inputs=[cins[0]], weights=cins[1:], name="conv_chain")
    cg = chimera.graph_fusion(runtime.Graph([cl, relu_layer([n, c2, hw_, hw_])], edges={(1, 0): (0, 0)}))
    assert len(cg.layers) == 1
    fl = cg.layers[0]
    func = ditto.build(common.describe_layer(fl), fl.schedule_tensors, "hip")
    assert func.sch.relu_out and func.sch.kind == "conv_chain"
    X, W1, W2 = oracle.make_conv_chain_inputs(n, c0, hw_, hw_, c1, c2, 3, 1, "float16", seed=8)
    want = oracle.np_round_to(oracle.conv_chain_f32(X, W1, W2, 1, 1, 0, 1, relu_mid=False, relu_out=True,
                                                    round_mid="float16"), "float16")
    for make in (runtime.create_graph_engine, runtime.create_hip_graph_engine):
        eng = make(cg, {fl.fingerprint: func}, "cuda:0")
        eng.set_inputs([to_dev(X, "float16")])
        eng.set_weight(fl, fl.weights[0], to_dev(W1, "float16"))
        eng.set_weight(fl, fl.weights[1], to_dev(W2, "float16"))
        eng.compile()
        assert eng._to_exe[0][0] is not func and eng._to_exe[0][0]._prepared is not None  # bound to these weights
        for _ in range(2):
            eng.run()
        torch.cuda.synchronize()
        got = eng.get_outputs()[0].float().cpu().numpy()
        assert (got >= 0).all() and (got == 0).mean() > 0.2
        mx, rel = errors(got, want)
        assert mx <= 1e-2 and rel <= 1e-3, (mx, rel)
        # new weights through set_weight are repacked at the next compile
        eng.set_weight(fl, fl.weights[1], to_dev(W2 * 0.5, "float16"))
        eng.run()
        torch.cuda.synchronize()
        half = oracle.np_round_to(oracle.conv_chain_f32(X, W1, oracle.np_round_to(W2 * 0.5, "float16"), 1, 1, 0, 1,
                                                        relu_mid=False, relu_out=True, round_mid="float16"), "float16")
        assert errors(eng.get_outputs()[0].float().cpu().numpy(), half)[1] <= 1e-3


def test_captured_conv_chain_survives_growth_of_the_shared_workspace(oracle):
    """A HIP graph that captured a conv chain call keeps replaying correctly after a later, larger chain made
    the shared per-device workspace grow: buffers that were handed out are never freed, and a built function
    owns its workspace."""
    import numpy as np

    from ditto_amd import chain
    from tests.gpu_util import errors, to_dev

    dev = "cuda:0"
    X, W1, W2 = oracle.make_conv_chain_inputs(2, 16, 24, 24, 32, 48, 3, 1, "float16", seed=2)
    x, w1, w2 = (to_dev(t, "float16") for t in (X, W1, W2))
    y = torch.zeros(2, 48, 24, 24, device=dev, dtype=torch.float16)
    chain.run_conv_chain(x, w1, w2, y)  # warm-up: sizes the shared workspace (1 MiB floor)
    torch.cuda.synchronize()
    want = y.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        chain.run_conv_chain(x, w1, w2, y)
    before = chain._WORKSPACES[torch.device(dev)][-1].data_ptr()
    # a chain whose repacked weights exceed the floor: the shared workspace grows
    bx = torch.zeros(1, 512, 8, 8, device=dev, dtype=torch.float16)
    bw1 = torch.zeros(256, 512, 3, 3, device=dev, dtype=torch.float16)
    bw2 = torch.zeros(32, 256, 1, 1, device=dev, dtype=torch.float16)
    by = torch.zeros(1, 32, 8, 8, device=dev, dtype=torch.float16)
    chain.run_conv_chain(bx, bw1, bw2, by)
    torch.cuda.synchronize()
    bufs = chain._WORKSPACES[torch.device(dev)]
    assert bufs[-1].data_ptr() != before and any(b.data_ptr() == before for b in bufs)  # grown, old one kept
    junk = [torch.full((1 << 20,), 0xAB, dtype=torch.uint8, device=dev) for _ in range(8)]  # would reuse a freed block
    for it in range(3):
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), it
    del junk


def test_specialised_conv_chain_notices_other_and_updated_weights(oracle):
    """A function bound to fixed weights (``specialize``) runs the fused kernel alone on the repacked copy it made.
    It must not take for its own (a) new weight tensors that the allocator placed at the addresses of the bound
    ones, nor (b) the bound tensors after an in-place update; the graph-replay engine records again after (b)."""
    import numpy as np

    from ditto_amd import chimera
    from ditto_amd.auto_compute.nn import functional as F
    from tests.gpu_util import errors, to_dev

    n, c0, hw_, c1, c2 = 4, 64, 28, 64, 256  # (a shape that runs on the row pipeline: repacked W1 in the workspace)
    cins, couts = F.Conv3x3Conv1x1(n, c0, hw_, hw_, c1, c2)
    cl = ac.layer([couts[0].op], inputs=[cins[0]], weights=cins[1:], name="conv_chain")
    func = ditto.build(common.describe_layer(cl), cl.schedule_tensors, "hip")
    X, W1, W2 = oracle.make_conv_chain_inputs(n, c0, hw_, hw_, c1, c2, 3, 1, "float16", seed=11)
    W1b = oracle.np_round_to(W1 * 0.5, "float16")
    ref = lambda w1: oracle.np_round_to(oracle.conv_chain_f32(X[:1], w1, W2, 1, 1, 0, 1, round_mid="float16"), "float16")
    want_a, want_b = ref(W1), ref(W1b)
    assert errors(want_a, want_b)[1] > 0.1  # the two weight sets are told apart easily
    x = to_dev(X, "float16")
    y = torch.empty(n, c2, hw_, hw_, device=x.device, dtype=torch.float16)

    def check(f, w1, w2, want):
        y.fill_(float("nan"))
        f(x, w1, w2, y)
        torch.cuda.synchronize()
        mx, rel = errors(y[:1].float().cpu().numpy(), want)
        assert mx <= 1e-2 and rel <= 1e-3, (mx, rel)

    # (a) the bound tensors go out of the caller's hands; same-size tensors with other values take their place
    w1, w2 = to_dev(W1, "float16"), to_dev(W2, "float16")
    f = func.specialize(w1, w2)
    check(f, w1, w2, want_a)
    p1, p2 = w1.data_ptr(), w2.data_ptr()
    del w1, w2
    w1n, w2n = to_dev(W1b, "float16"), to_dev(W2, "float16")
    # (the function keeps the bound tensors alive, so the allocator cannot hand their addresses out again)
    assert w1n.data_ptr() != p1 and w2n.data_ptr() != p2
    check(f, w1n, w2n, want_b)
    check(f, w1n, w2n, want_b)  # bound to the new ones now: prepared path
    assert f._is_prepared(w1n, w2n)
    # (b) in-place update of the bound weights
    w1n.copy_(to_dev(W1, "float16"))
    assert not f._is_prepared(w1n, w2n)
    check(f, w1n, w2n, want_a)
    assert f._is_prepared(w1n, w2n)
    # a view of the bound memory is the bound weights
    assert f._is_prepared(w1n.view(c1, c0, 3, 3), w2n.detach())
    # both engines, weights updated in place between runs
    for make in (runtime.create_graph_engine, runtime.create_hip_graph_engine):
        eng = make(runtime.Graph([cl]), {cl.fingerprint: func}, "cuda:0")
        eng.set_inputs([x])
        ew1, ew2 = to_dev(W1, "float16"), to_dev(W2, "float16")
        eng.set_weight(cl, cl.weights[0], ew1)
        eng.set_weight(cl, cl.weights[1], ew2)
        eng.compile()
        eng.run()
        torch.cuda.synchronize()
        assert errors(eng.get_outputs()[0][:1].float().cpu().numpy(), want_a)[1] <= 1e-3
        ew1.mul_(0.5)  # exact in fp16: now W1b
        eng.run()
        torch.cuda.synchronize()
        assert errors(eng.get_outputs()[0][:1].float().cpu().numpy(), want_b)[1] <= 1e-3, make.__name__
