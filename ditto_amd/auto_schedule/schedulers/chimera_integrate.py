"""Choice of the kernel variant of a BMM chain: analytic filter, measurement, tuning log.

Counterpart of python/ditto/auto_schedule/schedulers/chimera_integrate.py.  The reference
searches a 10-dimensional CUDATensorizeParam space (:99-123) with an analytic
capacity / traffic filter (:229-295: over-capacity -> 1e10, else waves x staged kilobytes /
shared-memory bandwidth), measures the survivors and appends one JSON line per measurement to
``chimera_<log_file>`` (:326-333); ``auto_schedule_build_tasks`` later keeps, per workload key,
the entry with the smallest ``value`` (:527-537).

Here the space is the library's handful of kernel variants for the shape
(``ditto_bmm_chain_select_tile`` with ``tile_variant`` forced), the filter has the same two
parts, and the log keeps the reference's line format
``{"wkl_key": ..., "entry": {"record": {...}, "value": <ms>}}`` with the tile description
as the record, so a log written here can be re-read by ``load_best_records`` / ``best_variant``
and fed back through ``run_bmm_chain(..., tile_variant=...)``.
"""
import copy
import ctypes
import json
import os

from ... import _lib, chain
from ...hardware import query_hw_param

# kernel codes of the fp16/bf16 chain: four waves x 32 | 64 rows, eight waves x 32 rows (staggered phases,
# software pipelined, on the 16x16x32 MFMA with 256-row workgroups, the same with 384-row workgroups for the
# first row blocks: the library refuses these two unless B is stored [L][K]), four waves with 64-row workgroups on
# the 16x16x32 MFMA (a wave owns 16 rows and all keys | 32 rows and half the keys; head size up to 64)
FP_VARIANT_CODES = (1, 2, 8, 9, 6, 7, 4, 5)


# int8 chain: 8000 + 10 * (row tiles of 32 per workgroup) + depth of the ring of staged weight chunks
I8_VARIANTS = (8012, 8014, 8022, 8023)


class TuneEntry:
    """One measurement: ``record`` (the tile description, JSON-able) and ``value`` (ms)."""

    def __init__(self, record, value):
        self.record = record
        self.value = value

    def to_json(self):
        return {"record": self.record, "value": self.value}


def make_tile_variant_space(desc):
    """Variants of the library that can run ``desc`` (capacity filter: the library rejects the
    ones whose tile does not fit), as a list of tile descriptions."""
    lib = _lib.load()
    tile = _lib.TileParam()
    auto = copy.copy(desc)
    auto.tile_variant = 0
    _lib.check(lib.ditto_bmm_chain_select_tile(ctypes.byref(auto), ctypes.byref(tile)))
    space = []
    if desc.in_dtype in (_lib.F16, _lib.BF16):
        for q in FP_VARIANT_CODES:
            d = copy.copy(desc)
            d.tile_variant = tile.head_pad * 10 + q
            t = _lib.TileParam()
            if lib.ditto_bmm_chain_select_tile(ctypes.byref(d), ctypes.byref(t)) == _lib.OK:
                space.append(t.to_json())
    elif desc.in_dtype == _lib.I8:
        for variant in I8_VARIANTS:
            d = copy.copy(desc)
            d.tile_variant = variant
            t = _lib.TileParam()
            if lib.ditto_bmm_chain_select_tile(ctypes.byref(d), ctypes.byref(t)) == _lib.OK:
                space.append(t.to_json())
    else:
        space.append(tile.to_json())
    return space


def evaluate_param_hip(desc, tile, hw_param=None):
    """Analytic score of a tile (lower is better; 1e10 = over capacity), the shape of the
    reference's filter: rounds of workgroups over the CUs x bytes each workgroup stages through
    LDS / LDS bandwidth, plus the MFMA time of a round.  It ranks variants; it is not a time."""
    hw = hw_param or query_hw_param("gpu.hip.MI355X")
    if tile["lds_bytes"] > hw.shared_memory_per_group_kb * 1024:
        return 1e10
    groups = hw.num_groups
    per_cu = max(1, int(hw.shared_memory_per_group_kb * 1024 // max(tile["lds_bytes"], 1)))
    per_cu = min(per_cu, 2 if tile["block_threads"] <= 256 else 1)
    rounds = -(-tile["grid_x"] // (groups * per_cu))
    elem = 1 if desc.in_dtype == _lib.I8 else (4 if desc.in_dtype == _lib.F32 else 2)
    staged = desc.L * (desc.K + desc.N) * elem                     # B and C tiles of one workgroup
    flops = 2.0 * tile["block_m"] * desc.L * (desc.K + desc.N)     # of one workgroup
    lds_s = staged / (hw.shared_memory_bandwidth_gbs * 1e9 / groups)
    mfma_s = flops * per_cu / (2.5e15 / groups)
    return rounds * max(lds_s, mfma_s)


def _log(log_file, wkl_key, entry):
    with open(log_file, "a") as flog:
        print(json.dumps({"wkl_key": wkl_key, "entry": entry.to_json()}), file=flog, flush=True)


def select_tile_variant(wkl_key, log_file, A, B, C, F, inter_op="softmax", softmax_scale=1.0, top=3,
                        min_repeat_ms=50):
    """Measure the ``top`` analytically best variants for these operands, append every measurement
    to ``log_file`` and return the best ``TuneEntry``."""
    import torch

    desc = chain.bmm_chain_desc(A, B, C, F, inter_op, softmax_scale)
    space = sorted(make_tile_variant_space(desc), key=lambda t: evaluate_param_hip(desc, t))[:max(1, top)]
    best = None
    for tile in space:
        d = copy.copy(desc)
        d.tile_variant = tile["variant"]
        call = lambda: chain.run_bmm_chain(A, B, C, F, desc=d)
        call()
        torch.cuda.synchronize()
        n = 1
        while True:
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                call()
            e1.record()
            e1.synchronize()
            ms = e0.elapsed_time(e1)
            if ms >= min_repeat_ms or n >= 1 << 20:
                break
            n = max(n + 1, int(n * max(1.5, min_repeat_ms / max(ms, 1e-3) * 1.05)))
        entry = TuneEntry(tile, ms / n)
        _log(log_file, wkl_key, entry)
        if best is None or entry.value < best.value:
            best = entry
    return best


def load_best_records(log_file):
    """{wkl_key: entry} keeping the smallest ``value`` per key (chimera_integrate.py:527-537)."""
    params = {}
    if not os.path.exists(log_file):
        return params
    with open(log_file, "r") as fin:
        for line in fin:
            line = line.strip()
            if not line:
                continue
            obj = json.loads(line)
            if obj["wkl_key"] not in params or obj["entry"]["value"] < params[obj["wkl_key"]]["value"]:
                params[obj["wkl_key"]] = obj["entry"]
    return params


def best_variant(log_file, wkl_key, default=0):
    """Variant id recorded as best for ``wkl_key`` (``default`` = the library's table if unseen)."""
    entry = load_best_records(log_file).get(wkl_key)
    return entry["record"]["variant"] if entry else default


def workload_key(desc):
    """A stable key for a chain shape (the reference keys on the layer fingerprint)."""
    return "bmm_chain/dt%d/i%d/l%d/b%d/m%d/n%d/k%d/l%d" % (desc.in_dtype, desc.inter_op, desc.b_layout, desc.batch,
                                                         desc.M, desc.N, desc.K, desc.L)


def auto_schedule_bmm_chain_hip(key, log_file, A, B, C, F, inter_op="softmax", softmax_scale=1.0):
    """Tune once per key, then reuse the log: returns the variant id to pass as ``tile_variant``."""
    known = best_variant(log_file, key, default=None)
    if known is not None:
        return known
    return select_tile_variant(key, log_file, A, B, C, F, inter_op, softmax_scale).record["variant"]


# ---- conv -> conv chains: the same measurement and log over the conv kernel families ------------
# family ids of ``ditto_conv_chain_desc.tile_variant`` (include/ditto_chain.h): general kernel with a 1x1 second
# convolution, general kernel with the second convolution through LDS, W2 resident in LDS, the two row pipelines;
# depthwise: the tile kernels and the two row-streaming ones
CONV_FAMILY_IDS = (3000, 3500, 3600, 3700, 3800, 4000, 4024, 4025)


def make_conv_tile_variant_space(desc):
    """Kernels of the library that can run the conv chain ``desc``: one tile description per family that accepts
    it (the library refuses the others), each carrying the exact variant id the family resolves to."""
    lib = _lib.load()
    space, seen = [], set()
    for fam in (0,) + CONV_FAMILY_IDS:
        d = copy.copy(desc)
        d.tile_variant = fam
        t = _lib.TileParam()
        if lib.ditto_conv_chain_select_tile(ctypes.byref(d), ctypes.byref(t)) == _lib.OK and t.variant not in seen:
            seen.add(t.variant)
            space.append(t.to_json())
    return space


def conv_workload_key(desc):
    return "conv_chain/dt%d/o%d/i%d/r%d/n%d/c%d/h%d/w%d/c%d/k%d/p%d/s%d/c%d/k%d/p%d/g%d" % (
        desc.in_dtype, desc.out_dtype, desc.inter_op, desc.relu_out, desc.N, desc.C0, desc.H, desc.W, desc.C1, desc.R1,
        desc.pad1, desc.stride1, desc.C2, desc.R2, desc.pad2, max(1, desc.groups1))


def select_conv_tile_variant(wkl_key, log_file, X, W1, W2, Y, pad1=1, stride1=1, pad2=0, stride2=1, inter_op="cast",
                             relu_out=False, groups1=1, min_repeat_ms=50):
    """Measure every kernel that can run this conv chain with its weights prepared once (the fused kernel alone is
    timed, as the reference times a function whose weights the host has packed), append every measurement to
    ``log_file`` and return the best ``TuneEntry``."""
    import torch

    desc = chain.conv_chain_desc(X, W1, W2, Y, pad1, stride1, pad2, stride2, inter_op, relu_out, groups1)
    best = None
    for tile in make_conv_tile_variant_space(desc):
        d = copy.copy(desc)
        d.tile_variant = tile["variant"]
        ws = chain.prepare_conv_chain(d, W1, W2) if chain.conv_chain_workspace_bytes(d) else None
        if ws is not None:
            call = lambda: chain.run_conv_chain(X, W1, W2, Y, desc=d, workspace=ws, prepared=True)
        else:
            call = lambda: chain.run_conv_chain(X, W1, W2, Y, desc=d)
        call()
        torch.cuda.synchronize()
        n = 1
        while True:
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                call()
            e1.record()
            e1.synchronize()
            ms = e0.elapsed_time(e1)
            if ms >= min_repeat_ms or n >= 1 << 20:
                break
            n = max(n + 1, int(n * max(1.5, min_repeat_ms / max(ms, 1e-3) * 1.05)))
        entry = TuneEntry(tile, ms / n)
        _log(log_file, wkl_key, entry)
        if best is None or entry.value < best.value:
            best = entry
    return best


def auto_schedule_conv_chain_hip(key, log_file, X, W1, W2, Y, **kw):
    """Tune once per key, then reuse the log: returns the variant id to pass as ``tile_variant``."""
    known = best_variant(log_file, key, default=None)
    if known is not None:
        return known
    return select_conv_tile_variant(key, log_file, X, W1, W2, Y, **kw).record["variant"]


# ---- layer-level entry points (chimera_integrate.py:452-556 of the reference) -------------------
class AttentionSchedule:
    """What scheduling a ``multi_head_attention_mma_layer`` yields: the layer, the module that runs
    it and the kernel variant chosen for its shape (0: the library's table)."""

    def __init__(self, layer, module, tile_variant=0):
        self.layer = layer
        self.module = module
        self.tile_variant = int(tile_variant)


def _attention_module(layer, schedule_option=None):
    from ...auto_compute.nn.module import MultiHeadAttentionMMA

    op = layer.ops[0]
    if getattr(op, "kind", None) != "mha":
        raise ValueError("layer %s is not a multi-head attention layer" % layer.name)
    a = op.attrs
    mi, ni, ki = a.get("mma", (16, 16, 16))
    return MultiHeadAttentionMMA(a["num_heads"], a["num_heads"] * a["head_dim"], op.output(0).dtype,
                                 a.get("acc_dtype", "float32"), mi, ni, ki, scale=a["scale"])


def _attention_operands(layer, module, dev="cuda:0"):
    """Synthetic operands of the layer's shape for measurement: the packed projection and the
    output, and the per-head views the kernel is called with."""
    import torch

    dt = {"float16": torch.float16, "bfloat16": torch.bfloat16}[layer.inputs[0].dtype]
    qkv = torch.randn(tuple(layer.inputs[0].shape), device=dev).to(dt)
    out = torch.empty(tuple(layer.ops[0].output(0).shape), dtype=dt, device=dev)
    q, k, v = module.head_views(qkv)
    batch, M = qkv.shape[0], qkv.shape[1]
    o = out.view(batch, M, module.num_heads, module.model_k).permute(0, 2, 1, 3)
    return q, k, v, o


def chimera_log_file(schedule_option):
    """The reference writes its measurements to ``chimera_<log_file>`` (:326-333, :530)."""
    head, tail = os.path.split(schedule_option.log_file)
    return os.path.join(head, "chimera_" + tail)


def auto_schedule(wkl_key, layer, schedule_option):
    """Measure the kernel variants for the layer's shape and log them (:452-512)."""
    module = _attention_module(layer, schedule_option)
    q, k, v, o = _attention_operands(layer, module)
    return select_tile_variant(wkl_key, chimera_log_file(schedule_option), q, k, v, o, "softmax", module.scale)


def auto_schedule_tasks(tasks, schedule_option):
    """``tasks``: OrderedDict[workload key, [layers]]; tunes the first layer of every key (:515-519)."""
    params = []
    for wkl_key, layers in tasks.items():
        entry = auto_schedule(wkl_key, layers[0], schedule_option)
        params.append({"wkl_key": wkl_key, "entry": entry.to_json()})
    return params


def auto_schedule_build_tasks(tasks, schedule_option):
    """{workload key: (schedule, schedule_tensors)} from the best logged record of every task
    (:527-556); a task without a record gets the library's own choice."""
    best = load_best_records(chimera_log_file(schedule_option))
    schedules = {}
    for k, layers in tasks.items():
        layer = layers[0]
        variant = best[k]["record"]["variant"] if k in best else 0
        schedules[k] = (AttentionSchedule(layer, _attention_module(layer, schedule_option), variant),
                        layer.schedule_tensors)
    return schedules
