"""Host-side mirror of the reference's descriptor API (no GPU): pattern classification,
DAG partition, chain recognition, error behaviour.  Expected values restate what the
reference's own tests / drivers show (python_test/auto_tensorize/test_pattern.py:9-66,
benchmark/chimera/cuda/bmm_softmax_bmm_cuda.py:158-236, src/auto_tensorize/hyper_fusion.cc:51-216)."""
import pytest

import ditto_amd as ditto
from ditto_amd import auto_compute as ac
from ditto_amd import auto_tensorize as at
from ditto_amd import hardware as hw
from ditto_amd import te

F = ac.nn.functional


def _describe(ins, outs, attach_pos=3):
    A, B, C = ins
    (Fo,) = outs
    E_frag = Fo.op.input_tensors[0]
    mid, C_ext = E_frag.op.input_tensors
    D_frag = mid.op.input_tensors[0]
    b, m, n, mi, ni = E_frag.op.axis
    rlo, rli = E_frag.op.reduce_axis
    fuse_choice = at.fusion_choice(D_frag.op, E_frag.op, [b, m, n, rlo, mi, ni, rli], attach_pos)
    first = at.cuda_wmma(M=16, N=16, K=16, in_dtype="float16", out_dtype="float32", scope="shared")
    second = at.cuda_wmma(M=16, N=16, K=16, in_dtype="float16", out_dtype="float32", scope="global")
    c1 = at.intrinsic_match(D_frag, first, ["InnerMost", "SameRange"])[0]
    c2 = at.intrinsic_match(E_frag, second, ["InnerMost", "SameRange"])[0]
    layer = ac.layer([Fo.op], inputs=[A, B, C])
    state = at.tensorize_hyper_fusion_state(
        layer, fuse_choice, {D_frag.op: at.match_info(c1, first), E_frag.op: at.match_info(c2, second)})
    return layer, state, D_frag, E_frag, (c1, c2)


def test_softmax_chain_partition_matches_reference():
    ins, outs = F.BatchGemmSoftmaxGemm(12, 512, 64, 64, 512, scale=0.125)
    layer, state, D_frag, E_frag, (c1, c2) = _describe(ins, outs)
    # bmm_softmax_bmm_cuda.py: prologues [[A_shared],[B_shared]], inter path [exp],
    # second prologue [[C_ext]], epilogue [F]
    assert [[o.name for o in v] for v in state.first_op_prologue] == [["A_shared"], ["B_shared"]]
    assert [o.name for o in state.inter_path] == ["exp"]
    assert [[o.name for o in v] for v in state.second_op_prologue] == [["C_ext"]]
    assert [o.name for o in state.epilogue] == ["F"]
    assert [iv.name for iv in state.fused_spatial_outer_iters] == ["b", "mo", "no"]
    assert [iv.name for iv in state.fused_reduce_outer_iters] == ["rlo"]
    assert [iv.name for iv in c1] == ["mi", "li", "rki"] and [iv.name for iv in c2] == ["mi", "ni", "rli"]
    # ones-column padding: ext_N = 2^ceil(log2(N/16 + 1)) * 16 (bmm_chain.py:72)
    assert E_frag.shape[2] * E_frag.shape[4] == 128
    assert layer.schedule_tensors[:3] == list(ins) and layer.schedule_tensors[3] is outs[0]
    assert "First op: D_frag" in state.summary() and "Inter Path:\n[exp ]" in state.summary(verbose=True)
    sch = at.tensorize_cuda(layer, state, hw.query_hw_param("gpu.cuda.A100"), at.cuda_tensorize_param())
    assert (sch.kind, sch.inter_op, sch.softmax_scale) == ("bmm_chain", "softmax", 0.125)
    assert sch.dims == dict(batch=12, M=512, N=64, K=64, L=512)


def test_gemm_chain_partition_and_relu():
    for relu, name in ((False, "cast"), (True, "relu")):
        ins, outs = F.BatchGemmGemm(1, 512, 64, 64, 64, relu=relu)
        layer, state, *_ = _describe(ins, outs)
        assert [o.name for o in state.inter_path] == [name]
        sch = at.tensorize_hip(layer, state)
        assert (sch.kind, sch.inter_op) == ("bmm_chain", name)


def test_patterns():
    ins, outs = F.BatchGemmSoftmaxGemm(2, 64, 64, 64, 64)
    layer = ac.layer([outs[0].op], inputs=ins)
    pat = {op.name: at.GetOpPattern(op) for op in layer.all_ops if isinstance(op, te.ComputeOp)}
    assert pat["D_frag"] == at.PATTERN_CUBIC and pat["E_frag"] == at.PATTERN_CUBIC
    assert pat["exp"] == at.PATTERN_LOCAL and pat["A_shared"] == at.PATTERN_SHUFFLE
    # a contraction whose shared reduce extent is below SUBSTANTIAL (16) is not cubic
    x = te.placeholder([64, 8], "x")
    y = te.placeholder([8, 64], "y")
    r = te.reduce_axis([0, 8], "r")
    small = te.compute([64, 64], "small", "float32", "contract", lambda i, j: [(x, [i, r]), (y, [r, j])],
                       reduce_axes=[r])
    assert not at.IsCubic(small.op)
    cins, couts = F.Conv3x3Conv1x1(32, 64, 56, 56, 64, 256)
    clayer = ac.layer([couts[0].op], inputs=[cins[0]], weights=cins[1:])
    cpat = {op.name: at.GetOpPattern(op) for op in clayer.all_ops if isinstance(op, te.ComputeOp)}
    assert cpat["conv1"] == at.PATTERN_CUBIC and cpat["conv2_fact"] == at.PATTERN_CUBIC
    assert cpat["pad1"] == at.PATTERN_SHUFFLE and cpat["cast"] == at.PATTERN_LOCAL


def test_serial_fusion_state_and_validate():
    ins, outs = F.BatchGemmGemm(1, 96, 64, 64, 64)
    layer = ac.layer([outs[0].op], inputs=ins)
    sfs = at.build_serial_fusion_state(layer)
    assert (sfs.first_op.name, sfs.second_op.name) == ("D_frag", "E_frag")
    assert at.validate(sfs) == (True, "")
    # a layer with a single contraction is refused: "we only deal with 2 CUBIC ops"
    A = te.placeholder([1, 64, 64], "A", "float16")
    B = te.placeholder([1, 64, 64], "B", "float16")
    r = te.reduce_axis([0, 64], "r")
    one = te.compute([1, 64, 64], "mm", "float32", "contract", lambda b, i, j: [(A, [b, i, r]), (B, [b, r, j])],
                     reduce_axes=[r])
    with pytest.raises(ValueError, match="2 CUBIC ops"):
        at.build_serial_fusion_state(ac.layer([one.op], inputs=[A, B]))


def test_descriptor_errors():
    ins, outs = F.BatchGemmGemm(1, 96, 64, 64, 64)
    A, B, C = ins
    (Fo,) = outs
    E_frag = Fo.op.input_tensors[0]
    D_frag = E_frag.op.input_tensors[0].op.input_tensors[0]
    layer = ac.layer([Fo.op], inputs=ins)
    iters = list(E_frag.op.axis) + list(E_frag.op.reduce_axis)
    wm = at.cuda_wmma()
    mi = {D_frag.op: at.match_info(D_frag.op.axis[-2:], wm), E_frag.op: at.match_info(E_frag.op.axis[-2:], wm)}
    with pytest.raises(ValueError, match="attach_pos"):
        at.tensorize_hyper_fusion_state(layer, at.fusion_choice(D_frag.op, E_frag.op, iters, len(iters)), mi)
    with pytest.raises(ValueError, match="match_info"):
        at.tensorize_hyper_fusion_state(layer, at.fusion_choice(D_frag.op, E_frag.op, iters, 3),
                                        {D_frag.op: mi[D_frag.op]})
    # swapped contraction order: the "first" op is not a producer of the "second"
    with pytest.raises(ValueError):
        at.tensorize_hyper_fusion_state(layer, at.fusion_choice(E_frag.op, D_frag.op, iters, 3), mi)
    # shape divisibility is asserted by the builders (bmm_chain.py:34-38)
    with pytest.raises(AssertionError):
        F.BatchGemmGemm(1, 100, 64, 64, 64)
    # placeholders must be declared to the layer
    with pytest.raises(ValueError, match="not listed"):
        ac.layer([Fo.op], inputs=[A, B])
    with pytest.raises(ValueError):
        at.hip_mfma(16, 16, 16, "float16", "float32")
    with pytest.raises(KeyError):
        hw.query_hw_param("gpu.hip.NOPE")


def test_tensorize_param_and_hardware_tables():
    p = at.cuda_tensorize_param(warp_size=32, ty_size=4, tz_size=2, input_vector_len=4, serial_y=2, serial_z=1,
                                block_rx=8, warp_rx=4, block_ry=1, warp_ry=4, unroll_steps=512)
    assert p.to_json() == {"warp_size": 32, "ty_size": 4, "tz_size": 2, "input_vector_len": 4, "serial_y": 2,
                           "serial_z": 1, "block_rx": 8, "warp_rx": 4, "block_ry": 1, "warp_ry": 4,
                           "unroll_steps": 512}
    d = at.cuda_tensorize_param()
    assert (d.warp_size, d.ty_size, d.tz_size, d.input_vector_len, d.serial_y, d.serial_z, d.block_rx, d.block_ry,
            d.block_rz, d.warp_rx, d.warp_ry, d.warp_rz, d.unroll_steps) == (32, 4, 2, 4, 2, 1, 4, 1, 4, 1, 4, 1, 1500)
    v100 = hw.query_hw_param("gpu.cuda.V100")
    assert (v100.num_groups, v100.shared_memory_per_group_kb, v100.global_memory_bandwidth_gbs) == (80, 96, 750)
    mi = hw.query_hw_param("gpu.hip.MI355X")
    assert mi.num_groups == 256 and mi.shared_memory_per_group_kb == 160 and mi.global_memory_bandwidth_gbs == 8000


def test_conv_chain_recognition():
    ins, outs = F.conv_relu_conv(1, 64, 56, 56, 128, 3, 3, 64, 1, 1, 1, 0, 1, 1)
    layer = ac.layer([outs[0].op], inputs=[ins[0]], weights=ins[1:])
    sfs = at.build_serial_fusion_state(layer)
    n_, k_, p_, q_ = sfs.second_op.axis
    fc = at.fusion_choice(sfs.first_op, sfs.second_op, [n_, p_, q_, k_] + sfs.second_op.reduce_axis, 2)
    mfma = at.hip_mfma(32, 32, 16, "float16", "float32")
    state = at.tensorize_hyper_fusion_state(layer, fc, {sfs.first_op: at.match_info(sfs.first_op.axis[-1:], mfma),
                                                        sfs.second_op: at.match_info(sfs.second_op.axis[-1:], mfma)})
    assert [o.name for o in state.inter_path] == ["relu", "pad2"]
    sch = at.tensorize_hip(layer, state)
    assert sch.kind == "conv_chain" and sch.inter_op == "relu"
    assert sch.dims["C1"] == 128 and sch.dims["pad1"] == 1 and sch.dims["R2"] == 1
    func = ditto.build(sch, layer.schedule_tensors, "hip")
    assert func.entry_name == "default_function" and len(func.tensors) == 4


def test_multi_head_attention_views_map_onto_two_level_strides():
    # the head split / merge of nn/module/self_attention.py:46-73 as strides of the chain descriptor
    import torch
    from ditto_amd import auto_compute as ac, chain

    batch, heads, M, d = 4, 16, 128, 64
    hidden = heads * d
    mha = ac.nn.module.MultiHeadAttentionMMA(heads, hidden, in_dtype="float16")
    assert mha.name == "multi_head_attention_mma_layer" and ac.nn.module.is_self_attention_layer(mha)
    qkv = torch.zeros(batch, M, 3 * hidden, dtype=torch.float16)
    out = torch.zeros(batch, M, hidden, dtype=torch.float16)
    q, k, v = mha.head_views(qkv)
    assert q.shape == (batch, heads, M, d) and k.shape == (batch, heads, d, M) and v.shape == q.shape
    assert q.data_ptr() == qkv.data_ptr() and k.data_ptr() == qkv.data_ptr() + 2 * hidden
    desc = chain.bmm_chain_desc(q, k, v, out.view(batch, M, heads, d).permute(0, 2, 1, 3), "softmax", 0.125)
    assert (desc.batch, desc.batch_inner, desc.M, desc.K, desc.L, desc.N) == (batch * heads, heads, M, d, M, d)
    assert desc.b_layout == 1  # keys stay [L][K]
    assert (desc.a_batch_stride, desc.a_batch_stride_outer, desc.a_row_stride) == (d, M * 3 * hidden, 3 * hidden)
    assert (desc.f_batch_stride, desc.f_batch_stride_outer, desc.f_row_stride) == (d, M * hidden, hidden)
    tile = chain.select_tile(desc)  # valid for the library
    assert tile.head_pad == 64
    import pytest
    with pytest.raises(RuntimeError):
        mha.head_views(torch.zeros(batch, M, 3 * hidden + 8, dtype=torch.float16))


def test_tuning_log_format_and_best_record(tmp_path):
    # line format and "smallest value per key wins" of chimera_integrate.py:326-333, 527-537
    import json
    from ditto_amd.auto_schedule.schedulers import chimera_integrate as ci

    log = str(tmp_path / "chimera_log.txt")
    for key, variant, value in (("a", 641, 0.5), ("a", 648, 0.3), ("b", 1282, 2.0), ("a", 642, 0.4)):
        ci._log(log, key, ci.TuneEntry({"variant": variant}, value))
    lines = [json.loads(l) for l in open(log)]
    assert set(lines[0]) == {"wkl_key", "entry"} and set(lines[0]["entry"]) == {"record", "value"}
    best = ci.load_best_records(log)
    assert best["a"]["record"]["variant"] == 648 and best["b"]["value"] == 2.0
    assert ci.best_variant(log, "a") == 648 and ci.best_variant(log, "zzz") == 0
    assert ci.load_best_records(str(tmp_path / "missing")) == {}


def test_tile_variant_space_and_analytic_filter():
    import torch
    from ditto_amd import chain
    from ditto_amd.auto_schedule.schedulers import chimera_integrate as ci

    def desc(b, s, d):
        q = torch.zeros(b, s, d, dtype=torch.bfloat16)
        return chain.bmm_chain_desc(q, q.transpose(1, 2), q, torch.zeros_like(q), "softmax", 0.1)

    big = desc(64, 4096, 128)
    space = ci.make_tile_variant_space(big)
    assert sorted(t["variant"] for t in space) == [1281, 1282, 1286, 1287, 1288, 1289]
    assert all(t["lds_bytes"] <= 160 * 1024 for t in space)
    scores = {t["variant"]: ci.evaluate_param_hip(big, t) for t in space}
    assert all(0 < v < 1e10 for v in scores.values())
    assert scores[1282] <= scores[1281]          # 256-row workgroups stage half as much per row
    over = dict(space[0], lds_bytes=200 * 1024)
    assert ci.evaluate_param_hip(big, over) == 1e10
    # few row blocks: the 128-row variant needs fewer rounds than the 256-row ones leave idle CUs
    small = desc(8, 2048, 128)
    sc = {t["variant"]: ci.evaluate_param_hip(small, t) for t in ci.make_tile_variant_space(small)}
    assert min(sc, key=sc.get) in (1281, 1282, 1286, 1287, 1288, 1289)
    assert ci.workload_key(big) != ci.workload_key(small)


def test_conv_tile_variant_space():
    """Kernel families that can run a conv chain, as the tuner enumerates them (no device needed)."""
    import torch
    from ditto_amd import chain
    from ditto_amd.auto_schedule.schedulers import chimera_integrate as ci

    def desc(N, C0, H, W, C1, R1, C2, R2, groups=1, dt=torch.float16):
        x = torch.zeros(N, C0, H, W, dtype=dt)
        w1 = torch.zeros(C1, C0 // groups, R1, R1, dtype=dt)
        w2 = torch.zeros(C2, C1, R2, R2, dtype=dt)
        y = torch.zeros(N, C2, H, W, dtype=dt)
        return chain.conv_chain_desc(x, w1, w2, y, R1 // 2, 1, R2 // 2, 1, "cast", False, groups)

    fams = lambda d: sorted(t["variant"] // 100 * 100 for t in ci.make_conv_tile_variant_space(d))
    assert fams(desc(32, 64, 56, 56, 64, 3, 256, 1)) == [3000, 3700]          # conv3x3 -> conv1x1
    assert fams(desc(32, 64, 56, 56, 64, 1, 64, 3)) == [3500, 3600, 3800]     # conv1x1 -> conv3x3
    assert fams(desc(1, 128, 28, 28, 128, 3, 128, 3)) == [3500]               # conv3x3 -> conv3x3: the general kernel only
    space = ci.make_conv_tile_variant_space(desc(32, 32, 112, 112, 32, 3, 64, 1, groups=32))
    assert sorted(t["variant"] for t in space) == [4023, 4024]                 # depthwise, multiplier 1
    space = ci.make_conv_tile_variant_space(desc(32, 32, 112, 112, 512, 3, 64, 1, groups=32))
    assert sorted(t["variant"] for t in space) == [4022, 4025]                 # depthwise, multiplier 16
    a, b = desc(32, 64, 56, 56, 64, 3, 256, 1), desc(16, 64, 56, 56, 64, 3, 256, 1)
    assert ci.conv_workload_key(a) != ci.conv_workload_key(b)


def test_attention_layer_task_extraction_and_binding():
    """bert_inference.py:88-92 -- tasks keyed by layer fingerprint, attention layers bound to the
    chimera scheduler (chimera/task_binding.py:6-20), everything else to ansor."""
    from ditto_amd import auto_schedule, chimera, runtime

    mha = ac.nn.module.MultiHeadAttentionMMA(12, 768, "float16", "float32", scale=None)
    other = ac.nn.module.MultiHeadAttentionMMA(6, 768, "float16", "float32", scale=None)
    layer = mha.layer(2, 512)
    assert layer.name == "multi_head_attention_mma_layer" and ac.nn.module.is_self_attention_layer(layer)
    assert [tuple(t.shape) for t in layer.schedule_tensors] == [(2, 512, 2304), (2, 512, 768)]
    # same shapes, different head count: a different workload
    assert layer.fingerprint != other.layer(2, 512).fingerprint
    assert layer.fingerprint == mha.layer(2, 512).fingerprint
    ins, outs = ac.nn.functional.BatchGemmGemm(4, 64, 64, 64, 64, "float16", "float32")
    gemm = ac.layer([outs[0].op], inputs=ins, name="gemm_chain_layer")
    graph = chimera.graph_fusion(runtime.Graph([mha.layer(2, 512), gemm, mha.layer(2, 512)], outputs=[(2, 0)]))
    tasks = auto_schedule.extract_tasks_from_graph(graph)
    assert list(tasks) == [layer.fingerprint, gemm.fingerprint] and [len(v) for v in tasks.values()] == [2, 1]
    bound = chimera.task_binding(tasks)
    assert list(bound) == ["chimera", "ansor"]
    assert list(bound["chimera"]) == [layer.fingerprint] and list(bound["ansor"]) == [gemm.fingerprint]
    opt = auto_schedule.ScheduleOption("hip", log_file="x.log", device_name="gpu.hip.MI355X", mma_MI=32)
    assert opt.trials == 100 and opt.mma_in_dtype == "float16" and opt.mma_MI == 32 and opt.device is not None
    with pytest.raises(NotImplementedError):  # the generic scheduler is outside this package
        auto_schedule.retrieve_schedule_bound_tasks(bound, opt)
    with pytest.raises(ValueError):
        auto_schedule.get_tasks_scheduler_builder("tvm")


def test_retrieve_attention_schedule_from_log(tmp_path):
    """auto_schedule_build_tasks keeps the record with the smallest value per workload key
    (chimera_integrate.py:527-556) and falls back to the library's choice for an unseen key."""
    import json

    from ditto_amd import auto_schedule, chimera, runtime

    mha = ac.nn.module.MultiHeadAttentionMMA(12, 768, "float16", "float32", scale=None)
    graph = runtime.Graph([mha.layer(1, 512)])
    bound = chimera.task_binding(auto_schedule.extract_tasks_from_graph(graph))
    opt = auto_schedule.ScheduleOption("hip", log_file=str(tmp_path / "bert.log"))
    (key,) = bound["chimera"]
    sch, args = auto_schedule.retrieve_schedule_bound_tasks(bound, opt)[key]
    assert sch.tile_variant == 0 and [tuple(t.shape) for t in args] == [(1, 512, 2304), (1, 512, 768)]
    with open(tmp_path / "chimera_bert.log", "w") as f:
        for variant, value in ((641, 0.03), (648, 0.02), (642, 0.05)):
            print(json.dumps({"wkl_key": key, "entry": {"record": {"variant": variant}, "value": value}}), file=f)
    sch, _ = auto_schedule.retrieve_schedule_bound_tasks(bound, opt)[key]
    assert sch.tile_variant == 648 and sch.module.num_heads == 12 and sch.module.scale == 64 ** -0.5


def _reference_flow(ins, outs, in_dtype="float16", acc_dtype="float32"):
    """The flow of python_test/auto_tensorize/test_hyper_fusion.py:833-880: serial fusion state ->
    intrinsic match -> register_tensorize_axes (one flat list) -> build_fusion_choice -> state."""
    layer = ac.layer([outs[0].op], inputs=list(ins))
    sfs = at.build_serial_fusion_state(layer)
    op1, op2 = sfs.first_op, sfs.second_op

    def get_match_info(op, scope):
        packed = at.cuda_wmma(16, 16, 16, in_dtype, acc_dtype, scope)
        return at.match_info(at.intrinsic_match(op.output(0), packed, ["InnerMost", "SameRange"])[0], packed, impl="")

    first, second = get_match_info(op1, "shared"), get_match_info(op2, "global")
    sfs.register_tensorize_axes(list(first.axis) + list(second.axis))
    fuse_choice = at.build_fusion_choice(sfs, hw_param=hw.query_hw_param("gpu.cuda.V100"), dtype="float32",
                                         simple_mode=-1)
    state = at.tensorize_hyper_fusion_state(layer, fuse_choice, {op1: first, op2: second})
    return layer, sfs, fuse_choice, state


def test_build_fusion_choice_gives_the_order_the_reference_drivers_write_by_hand():
    # bmm_bmm_cuda.py:176 and bmm_softmax_bmm_cuda.py: [b, m, n, rlo, mi, ni, rli], 3
    for ins, outs in (F.BatchGemmSoftmaxGemm(12, 512, 64, 64, 512), F.BatchGemmGemm(1, 512, 64, 64, 64)):
        layer, sfs, fc, state = _reference_flow(ins, outs)
        E_frag = outs[0].op.input_tensors[0]
        b, m, n, mi, ni = E_frag.op.axis
        rlo, rli = E_frag.op.reduce_axis
        manual = at.fusion_choice(sfs.first_op, sfs.second_op, [b, m, n, rlo, mi, ni, rli], 3)
        assert fc.first_op is manual.first_op and fc.second_op is manual.second_op
        assert all(x is y for x, y in zip(fc.ordered_iters, manual.ordered_iters)) and len(fc.ordered_iters) == 7
        assert fc.attach_pos == 3
        assert fc.secondOpOuterIndices == [0, 1, 2, 5] and fc.secondOpOuterTilingFactors == [1, 1, 1, 1]
        assert [iv.name for iv in state.fused_spatial_outer_iters] == ["b", "mo", "no"]
        assert [iv.name for iv in state.fused_reduce_outer_iters] == ["rlo"]
        # every search mode names the same fusion (the kernels fix tiling and order themselves)
        for mode in (0, 1):
            other = at.build_fusion_choice(sfs, None, "float16", mode)
            assert all(x is y for x, y in zip(other.ordered_iters, fc.ordered_iters)) and other.attach_pos == 3
        sch = at.tensorize_cuda(layer, state, hw.query_hw_param("gpu.hip.MI355X"), at.cuda_tensorize_param())
        assert sch.kind == "bmm_chain"
    # errors: axes not registered, unknown dtype, unknown mode (CHECKs of hyper_fusion.cc:1978, 1988)
    ins, outs = F.BatchGemmGemm(1, 64, 64, 64, 64)
    sfs = at.build_serial_fusion_state(ac.layer([outs[0].op], inputs=ins))
    with pytest.raises(ValueError, match="register"):
        at.build_fusion_choice(sfs, None, "float32")
    sfs.register_tensorize_axes({sfs.second_op: list(sfs.second_op.axis[-2:]) + [sfs.second_op.reduce_axis[-1]]})
    with pytest.raises(ValueError, match="dtype"):
        at.build_fusion_choice(sfs, None, "complex64")
    with pytest.raises(ValueError, match="simple_mode"):
        at.build_fusion_choice(sfs, None, "float32", 7)
    with pytest.raises(ValueError, match="neither contraction"):
        sfs.register_tensorize_axes([te.reduce_axis([0, 16], "stranger")])


def test_build_fusion_choice_on_conv_chains():
    # the hand-written choices of conv3x3_conv1x1_cuda.py:211 ([b, no, p, mo, rlo, mi, ni, rli], 4) and
    # conv1x1_conv3x3_cuda.py:228 ([b, no, p, mo, rlo, mi, ni, rr, rs, rli], 4) have this shape: spatial loops
    # that are not tensorized, the outermost free reduce loop, tensorized spatial loops, the other reduce loops
    for builder, n_red in ((F.Conv3x3Conv1x1, 3), (F.Conv1x1Conv3x3, 3)):
        cins, couts = builder(2, 64, 56, 56, 64, 64)
        layer = ac.layer([couts[0].op], inputs=[cins[0]], weights=cins[1:])
        sfs = at.build_serial_fusion_state(layer)
        op2 = sfs.second_op
        n, k, p, q = op2.axis
        c2, r2, s2 = op2.reduce_axis
        sfs.register_tensorize_axes([q, k, c2])  # pixel x output channel x input channel tile
        fc = at.build_fusion_choice(sfs, hw.query_hw_param("gpu.hip.MI355X"), "float16")
        assert [iv.name for iv in fc.ordered_iters] == ["n", "p", "rr2", "k", "q", "rs2", "rc2"]
        assert fc.attach_pos == 2 and fc.ordered_iters[fc.attach_pos] is r2


def test_int8_chain_builder_and_recognition():
    # the ("80", "int8", "int32") row of bmm_bmm_cuda.py:273-288, with the middle result requantised
    ins, outs = F.BatchGemmGemm(1, 8192, 1024, 1024, 256, "int8", "int32", requant_scale=2.0 ** -10)
    assert [t.dtype for t in ins] == ["int8"] * 3 and outs[0].dtype == "int32"
    layer, sfs, fc, state = _reference_flow(ins, outs, "int8", "int32")
    assert [o.name for o in state.inter_path] == ["requant"] and [o.name for o in state.epilogue] == ["F"]
    sch = at.tensorize_cuda(layer, state, hw.query_hw_param("gpu.hip.MI355X"), at.cuda_tensorize_param())
    assert (sch.kind, sch.inter_op, sch.in_dtype, sch.acc_dtype, sch.out_dtype) == (
        "bmm_chain", "requant", "int8", "int32", "int32")
    assert sch.requant_scale == 2.0 ** -10 and not sch.scale_tensor
    assert sch.dims == dict(batch=1, M=8192, N=1024, K=1024, L=256)
    # per-column scales: a fourth input placeholder, in schedule_tensors order before the output
    ins, outs = F.BatchGemmGemm(2, 64, 64, 64, 128, "int8", "int32", scale_tensor=True)
    assert len(ins) == 4 and ins[3].shape == (128,) and ins[3].dtype == "float32"
    layer, sfs, fc, state = _reference_flow(ins, outs, "int8", "int32")
    sch = at.tensorize_hip(layer, state)
    assert sch.scale_tensor and [t.name for t in layer.schedule_tensors] == ["A", "B", "C", "scale", "F"]
    # the reference's own int8 chain: astype("int8") for the middle result and for F (bmm_bmm_cuda.py:116, :147)
    for relu in (False, True):
        ins, outs = F.BatchGemmGemm(1, 64, 64, 64, 64, "int8", "int32", relu=relu)
        assert outs[0].dtype == "int8"
        layer, sfs, fc, state = _reference_flow(ins, outs, "int8", "int32")
        sch = at.tensorize_hip(layer, state)
        assert (sch.kind, sch.inter_op, sch.in_dtype, sch.acc_dtype, sch.out_dtype) == (
            "bmm_chain", "relu" if relu else "cast", "int8", "int32", "int8")
    # tile_variant travels on the schedule
    ins, outs = F.BatchGemmGemm(64, 4096, 128, 128, 4096, "bfloat16", "float32")
    layer, sfs, fc, state = _reference_flow(ins, outs, "bfloat16")
    assert at.tensorize_hip(layer, state, tile_variant=1288).tile_variant == 1288


def test_graph_fusion_folds_relu_layers_into_the_producing_chain():
    from ditto_amd import chimera, runtime

    def chain_layer(relu_mid=False):
        ins, outs = F.BatchGemmGemm(2, 128, 64, 64, 128, relu=relu_mid)
        return ac.layer([outs[0].op], inputs=ins, name="gemm_chain")

    def relu_layer(shape, name="act"):
        x = te.placeholder(shape, "x", "float16")
        return ac.layer([F.ReLU(x).op], inputs=[x], name=name)

    l0, act, l1 = chain_layer(), relu_layer([2, 128, 64]), chain_layer(True)
    graph = runtime.Graph([l0, act, l1], edges={(1, 0): (0, 0), (2, 0): (1, 0)})
    assert chimera.is_act_layer(act) and not chimera.is_act_layer(l0) and not chimera.is_elem_layer(act)
    fused = chimera.graph_fusion(graph)
    assert [l.name for l in fused.layers] == ["gemm_chain_relu", "gemm_chain"]
    assert fused.edges == {(1, 0): (0, 0)} and fused.graph_outputs == [(1, 0)]
    assert [l.name for l in graph.layers] == ["gemm_chain", "act", "gemm_chain"]  # the input graph is untouched
    out_op = fused.layers[0].ops[0]
    assert out_op.kind == "relu_cast" and out_op.attrs["fused_activation"] == "relu"
    assert fused.layers[0].fingerprint != l0.fingerprint
    # the fused layer still describes and tensorizes as a chain, now with the output ReLU
    layer, sfs, fc, state = None, None, None, None
    fl = fused.layers[0]
    sfs = at.build_serial_fusion_state(fl)
    p = at.cuda_wmma(16, 16, 16, "float16", "float32", "global")
    infos = {op: at.match_info(at.intrinsic_match(op.output(0), p, ["InnerMost", "SameRange"])[0], p)
             for op in (sfs.first_op, sfs.second_op)}
    sfs.register_tensorize_axes([iv for mi in infos.values() for iv in mi.axis])
    state = at.tensorize_hyper_fusion_state(fl, at.build_fusion_choice(sfs, None, "float16"), infos)
    sch = at.tensorize_hip(fl, state)
    assert (sch.inter_op, sch.relu_out) == ("cast", True)
    # not fused: a ReLU whose input is also a graph output, one behind a softmax chain, a gelu, a residual add
    keep = runtime.Graph([l0, act], edges={(1, 0): (0, 0)}, outputs=[(0, 0), (1, 0)])
    assert chimera.graph_fusion(keep) is keep
    sins, souts = F.BatchGemmSoftmaxGemm(2, 128, 64, 64, 128)
    sl = ac.layer([souts[0].op], inputs=sins, name="attn_chain")
    g2 = runtime.Graph([sl, relu_layer([2, 128, 64])], edges={(1, 0): (0, 0)})
    assert chimera.graph_fusion(g2) is g2
    x = te.placeholder([2, 128, 64], "x", "float16")
    gelu = ac.layer([F.activation(x, "gelu").op], inputs=[x], name="gelu")
    g3 = runtime.Graph([l0, gelu], edges={(1, 0): (0, 0)})
    assert chimera.graph_fusion(g3) is g3
    a, b = te.placeholder([2, 128, 64], "a", "float16"), te.placeholder([2, 128, 64], "b", "float16")
    add = ac.layer([F.elementwise(a, b, "add").op], inputs=[a, b], name="residual")
    assert chimera.is_elem_layer(add)
    g4 = runtime.Graph([l0, add], edges={(1, 0): (0, 0)})
    assert chimera.graph_fusion(g4) is g4
    # a conv chain takes the ReLU too (its descriptor already has the output slot)
    cins, couts = F.Conv3x3Conv1x1(2, 16, 16, 16, 32, 48)
    cl = ac.layer([couts[0].op], inputs=[cins[0]], weights=cins[1:], name="conv_chain")
    g5 = chimera.graph_fusion(runtime.Graph([cl, relu_layer([2, 48, 16, 16])], edges={(1, 0): (0, 0)}))
    assert len(g5.layers) == 1 and g5.layers[0].ops[0].kind == "relu_cast" and len(g5.layers[0].weights) == 2


def test_the_reference_import_name_resolves():
    """``from ditto import auto_compute as ac`` etc. (the first lines of the reference's drivers) give the modules of
    this package."""
    import ditto
    import ditto.auto_tensorize as at_ref
    from ditto import auto_compute as ac_ref
    from ditto.auto_compute.nn.functional import BatchGemmSoftmaxGemmMMA  # noqa: F401
    from ditto.hardware.hw_param import hardware_param

    import ditto_amd
    assert ac_ref is ditto_amd.auto_compute and at_ref is ditto_amd.auto_tensorize
    assert hardware_param is ditto_amd.hardware.hardware_param and ditto.build is ditto_amd.build
    assert ditto.chimera is ditto_amd.chimera and ditto.runtime.Graph is ditto_amd.runtime.Graph
