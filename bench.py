#!/usr/bin/env python3
"""Benchmark of the fused operator chains on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-also] [--no-zero]

A "step" is one call of the fused chain on one batch of synthetic input that is already
resident in HBM.  The headline workload is the long-sequence BMM -> softmax -> BMM chain
(bf16, 64 x (4096 x 128)): the MFMA-bound configuration on which the ">= 50 % of dense MFMA
peak" target is stated.  The other configurations are timed briefly and reported under
"also".  One JSON line is printed.

Timing protocol: untimed warm-up calls until both W calls and 300 ms of device work are done (a
fresh device needs that long to reach its steady clocks), then exactly K calls between two HIP
events recorded on the launch stream, bracketed by device synchronisation.  Beside it,
``roofline.min_repeat_600ms_ms`` is the mean per call over a timed region grown to at least 600 ms,
the reference's ``time_evaluator(..., min_repeat_ms=600)`` rule
(benchmark/chimera/cuda/bmm_softmax_bmm_cuda.py:39).  FLOPs are the algorithmic ``2*batch*M*L*(K+N)`` (the reference counts
``batch*M*L*(K+N)`` MACs, benchmark/chimera/cpu/bmm_bmm_cpu.py:281); softmax, casts and
padding count zero.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks (dense)
PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "i8": 5000.0, "f32": 157.3}
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch come from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summaries under profiles/ (each counter
# scaled by what it reads for a plain copy of known size in the same run: FETCH_SIZE reads half of a copy's bytes on
# this device, factor 2.00, WRITE_SIZE all of them).  A summary belongs to the kernel variant named in its header
# ("tile variant N"): when the library picks another variant for the workload, or no summary exists, the figure
# would be stale and ``roofline.traffic`` is null.
def measured_traffic(name, variant):
    import glob
    import re

    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*__%s.txt" % name))):
        text = open(path).read()
        m = re.search(r"tile variant (\d+)", text)
        f = re.search(r"^FETCH_SIZE: .* scaled ([0-9.]+) MiB per launch", text, re.M)
        w = re.search(r"^WRITE_SIZE: .* scaled ([0-9.]+) MiB per launch", text, re.M)
        if m and f and w and int(m.group(1)) == int(variant):
            return int((float(f.group(1)) + float(w.group(1))) * 2 ** 20)
    return None


WORKLOADS = {
    # name: kind, dtype, dims
    "attn_bf16_b64_s4096_d128": dict(kind="softmax", dtype="bfloat16", batch=64, M=4096, N=128, K=128, L=4096,
                                     scale=128 ** -0.5, bound="mfma",
                                     desc="BMM-softmax-BMM, batch 4x16 heads, seq 4096, head dim 128, bf16"),
    "attn_f16_b96_s512_d64": dict(kind="softmax", dtype="float16", batch=96, M=512, N=64, K=64, L=512,
                                  scale=0.125, bound="hbm",
                                  desc="BMM-softmax-BMM, BERT-base: batch 8x12 heads, seq 512, head dim 64, fp16"),
    "gemm_chain_f16_b1_512x64x64x64": dict(kind="cast", dtype="float16", batch=1, M=512, N=64, K=64, L=64,
                                           scale=1.0, bound="hbm",
                                           desc="GEMM chain (A.B).D at the shape of the CPU plumbing case, fp16"),
    "gemm_chain_bf16_b64_4096x128x4096x128": dict(kind="cast", dtype="bfloat16", batch=64, M=4096, N=128, K=128,
                                                  L=4096, scale=1.0, bound="mfma",
                                                  desc="batched GEMM chain (A.B).D with the cast between, at the "
                                                       "long-sequence attention shape: the large GEMM-chain point"),
}
WORKLOADS.update({
    "conv_chain_f16_n32_c64_56x56_k64_k256": dict(
        kind="conv", dtype="float16", N=32, C0=64, H=56, W=56, C1=64, R=3, pad=1, stride=1, C2=256, bound="hbm",
        desc="conv3x3(64->64, s1 p1) -> conv1x1(64->256) on 32x56x56, NCHW fp16"),
    "conv1x1_conv3x3_f16_n32_c64_56x56_k64_k64": dict(
        kind="conv", dtype="float16", N=32, C0=64, H=56, W=56, C1=64, R=1, pad=0, stride=1, C2=64, R2=3, pad2=1,
        bound="mfma",
        desc="conv1x1(64->64) -> conv3x3(64->64, s1 p1) on 32x56x56, NCHW fp16 (the reference's ResNet-50 row)"),
    "dw3x3_conv1x1_f16_n32_c32_112x112_f16_k64": dict(
        kind="conv", dtype="float16", N=32, C0=32, H=112, W=112, C1=512, R=3, pad=1, stride=1, C2=64, groups=32,
        bound="mfma",  # 30.0 GFLOP over 77.2 MB: 389 FLOP/B, above the ridge of 312
        desc="depthwise conv3x3(32 channels x16, s1 p1) -> conv1x1(512->64) on 32x112x112, NCHW fp16 "
             "(the reference's MobileNet-V1 row)"),
    "dw3x3_conv1x1_f16_n32_c32_112x112_x1_k64": dict(
        kind="conv", dtype="float16", N=32, C0=32, H=112, W=112, C1=32, R=3, pad=1, stride=1, C2=64, groups=32,
        bound="hbm",
        desc="depthwise conv3x3(32 channels, multiplier 1, s1 p1) -> conv1x1(32->64) on 32x112x112, NCHW fp16 "
             "(MobileNet-V1's first depthwise-separable block)"),
    "gemm_chain_i8_8192x1024x256x1024": dict(
        kind="requant", dtype="int8", batch=1, M=8192, K=1024, L=256, N=1024, scale=2.0 ** -10, bound="hbm",
        desc="int8 A[8192,1024].B[1024,256] -> requantise(2^-10, RNE, saturate) -> .D[256,1024], int32 out"),
})
DEFAULT_WORKLOAD = "attn_bf16_b64_s4096_d128"
SHORT = {"bfloat16": "bf16", "float16": "f16", "int8": "i8", "float32": "f32"}


def flops_of(w):
    if w["kind"] == "conv":
        P = (w["H"] + 2 * w["pad"] - w["R"]) // w["stride"] + 1
        Q = (w["W"] + 2 * w["pad"] - w["R"]) // w["stride"] + 1
        R2 = w.get("R2", 1)
        P2, Q2 = P + 2 * w.get("pad2", 0) - R2 + 1, Q + 2 * w.get("pad2", 0) - R2 + 1
        c0g = w["C0"] // w.get("groups", 1)
        return 2.0 * w["N"] * (P * Q * c0g * w["C1"] * w["R"] * w["R"] + P2 * Q2 * w["C1"] * w["C2"] * R2 * R2)
    return 2.0 * w["batch"] * w["M"] * w["L"] * (w["K"] + w["N"])


def bytes_of(w):
    """Algorithmic bytes: every input read once, the output written once."""
    if w["kind"] == "conv":
        P = (w["H"] + 2 * w["pad"] - w["R"]) // w["stride"] + 1
        Q = (w["W"] + 2 * w["pad"] - w["R"]) // w["stride"] + 1
        R2 = w.get("R2", 1)
        P2, Q2 = P + 2 * w.get("pad2", 0) - R2 + 1, Q + 2 * w.get("pad2", 0) - R2 + 1
        return 2 * (w["N"] * w["C0"] * w["H"] * w["W"] + w["C1"] * (w["C0"] // w.get("groups", 1)) * w["R"] * w["R"]
                    + w["C2"] * w["C1"] * R2 * R2 + w["N"] * w["C2"] * P2 * Q2)
    if w["kind"] == "requant":
        return w["batch"] * (w["M"] * w["K"] + w["K"] * w["L"] + w["L"] * w["N"] + 4 * w["M"] * w["N"])
    eb = 2
    return eb * w["batch"] * (w["M"] * w["K"] + w["K"] * w["L"] + w["L"] * w["N"] + w["M"] * w["N"])


def make_call(w, dev, prepared=False, zero=False):
    """Synthetic inputs resident on the device and a zero-argument callable that runs one step.
    ``prepared`` (conv chains that take a workspace): the weights are repacked once, outside the
    step, as the reference's drivers are handed host-packed weights; the step is the fused kernel alone.
    ``zero`` (BMM chains): all-zero operands, the same instructions on data that toggles nothing."""
    import torch

    from ditto_amd import chain

    g = torch.Generator().manual_seed(0)
    if w["kind"] == "conv":
        x = torch.randn(w["N"], w["C0"], w["H"], w["W"], generator=g).half().to(dev)
        groups = w.get("groups", 1)
        w1 = (torch.randn(w["C1"], w["C0"] // groups, w["R"], w["R"], generator=g) * (0.3 if groups > 1 else 0.05)
              ).half().to(dev)
        R2, pad2 = w.get("R2", 1), w.get("pad2", 0)
        w2 = (torch.randn(w["C2"], w["C1"], R2, R2, generator=g) * 0.05).half().to(dev)
        P = (w["H"] + 2 * w["pad"] - w["R"]) // w["stride"] + 1 + 2 * pad2 - R2 + 1
        Q = (w["W"] + 2 * w["pad"] - w["R"]) // w["stride"] + 1 + 2 * pad2 - R2 + 1
        y = torch.empty(w["N"], w["C2"], P, Q, dtype=torch.float16, device=dev)
        desc = chain.conv_chain_desc(x, w1, w2, y, w["pad"], w["stride"], pad2, 1, "cast", False, groups)
        if prepared:
            ws = chain.prepare_conv_chain(desc, w1, w2)
            return (lambda: chain.run_conv_chain(x, w1, w2, y, desc=desc, workspace=ws, prepared=True)), desc
        return (lambda: chain.run_conv_chain(x, w1, w2, y, desc=desc)), desc
    if w["kind"] == "requant":
        a = torch.randint(-127, 128, (w["M"], w["K"]), generator=g, dtype=torch.int8).to(dev)
        b = torch.randint(-127, 128, (w["K"], w["L"]), generator=g, dtype=torch.int8).to(dev)
        d = torch.randint(-127, 128, (w["L"], w["N"]), generator=g, dtype=torch.int8).to(dev)
        scale = torch.full((w["L"],), w["scale"], dtype=torch.float32, device=dev)
        e = torch.empty(w["M"], w["N"], dtype=torch.int32, device=dev)
        desc = chain.bmm_chain_desc(a, b, d, e, "requant")
        return (lambda: chain.run_bmm_chain(a, b, d, e, aux=scale, desc=desc)), desc
    dt = {"bfloat16": torch.bfloat16, "float16": torch.float16}[w["dtype"]]
    std = 1.0 if w["kind"] == "softmax" else 0.25
    a = (torch.randn(w["batch"], w["M"], w["K"], generator=g) * std).to(dt).to(dev)
    c = (torch.randn(w["batch"], w["L"], w["N"], generator=g) * std).to(dt).to(dev)
    if w["kind"] == "softmax":
        # keys are stored [batch, L, K]; the chain's B operand is the transposed view
        b = torch.randn(w["batch"], w["L"], w["K"], generator=g).to(dt).to(dev).transpose(1, 2)
    else:
        b = (torch.randn(w["batch"], w["K"], w["L"], generator=g) * std).to(dt).to(dev)
    if zero:
        a.zero_(), b.zero_(), c.zero_()
    f = torch.empty(w["batch"], w["M"], w["N"], dtype=dt, device=dev)
    desc = chain.bmm_chain_desc(a, b, c, f, w["kind"], w["scale"])
    return (lambda: chain.run_bmm_chain(a, b, c, f, desc=desc)), desc


def time_gpu(w, steps, warmup, dev, prepared=False, long_run=False):
    """(ms per step over the synchronised wall clock, ms per launch from HIP events around the eager
    loop, ms per launch from a graph replay of the same loop)."""
    import torch

    from ditto_amd import chain

    call, desc = make_call(w, dev, prepared)
    warm_up(call, warmup)
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        call()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = e0.elapsed_time(e1) / steps
    tile = chain.select_tile(desc).to_json()
    return wall_ms, ev_ms, graph_ms(call, steps), tile, (min_repeat_ms(call) if long_run else None)


WARMUP_MIN_S = 0.3


def warm_up(call, warmup):
    """At least ``warmup`` calls and at least WARMUP_MIN_S seconds of back-to-back device work."""
    import torch

    done, t0 = 0, time.perf_counter()
    while done < max(warmup, 1) or time.perf_counter() - t0 < WARMUP_MIN_S:
        for _ in range(max(warmup, 1)):
            call()
        torch.cuda.synchronize()
        done += max(warmup, 1)


def min_repeat_ms(call, min_ms=600.0):
    """Mean ms per call over a timed region of at least ``min_ms`` (the number of calls is grown until
    the region is long enough: TVM's ``min_repeat_ms`` rule)."""
    import torch

    n = 8
    while True:
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            call()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1)
        if ms >= min_ms or n >= (1 << 22):
            return ms / n
        n = max(n + 1, int(n * max(1.5, min_ms / max(ms, 1e-3) * 1.05)))


def graph_ms(call, steps):
    """ms per step with the `steps` launches recorded once into a HIP graph and replayed: the
    device-side duration of a step without the host's per-launch cost (which, for the
    configurations that finish in tens of microseconds, is of the same order as the kernel).
    None if the capture fails."""
    import torch

    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(steps):
                call()
        t0 = time.perf_counter()
        g.replay()
        torch.cuda.synchronize()
        # the capture leaves the device idle for a while: replay for about WARMUP_MIN_S first (a graph of a few
        # steps is otherwise timed on clocks that are still coming up), then time as many replays again
        reps = max(1, int(WARMUP_MIN_S / max(time.perf_counter() - t0, 1e-6)))
        for _ in range(reps):
            g.replay()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (steps * reps)
    except Exception:  # capture unsupported: the eager figure stands alone
        torch.cuda.synchronize()
        return None


def cpu_baseline(w, budget_s=10.0, pool=24):
    """The fused CPU loop nest (the checker's restatement of the reference's TensorizeCPU nest)
    on a bounded sample of the same workload: single batch entries of the chain, one call each,
    cycling over ``pool`` distinct pre-generated entries (so operands are not cache-resident from
    the previous call) until ``budget_s`` seconds of CPU time are used.  fp32 arithmetic, OpenMP
    over the host cores."""
    import numpy as np

    from oracle import oracle as orc

    rng = np.random.default_rng(0)
    M, N, K, L = w["M"], w["N"], w["K"], w["L"]
    per_entry = 2.0 * M * L * (K + N)
    pool = max(2, min(pool, int(2e9 // (4 * (M * K + K * L + L * N)))))
    entries = [(rng.standard_normal((1, M, K), dtype=np.float32), rng.standard_normal((1, K, L), dtype=np.float32),
                rng.standard_normal((1, L, N), dtype=np.float32)) for _ in range(pool)]
    out = np.empty((1, M, N), dtype=np.float32)
    inter = "softmax" if w["kind"] == "softmax" else w["kind"]
    run = lambda e: orc.bmm_chain_fused_f32(e[0], e[1], e[2], inter=inter, scale=w["scale"], mb=48, lb=256,  # noqa: E731
                                            out=out)
    run(entries[0])  # untimed: warms the thread pool and the code
    done, elapsed = 0, 0.0
    while elapsed < budget_s and done < 200000:
        e = entries[(done + 1) % pool]
        t0 = time.perf_counter()
        run(e)
        elapsed += time.perf_counter() - t0
        done += 1
    out = {
        "value": per_entry * done / elapsed / 1e12,
        "unit": "TFLOP/s",
        "cores": orc.num_threads(),
        "kind": "port",
        "sample": "%d single-batch-entry calls of the same chain (M=%d, L=%d, K=%d, N=%d) in fp32 through the "
                  "fused CPU loop nest (oracle_bmm_chain_fused_f32), cycling over %d distinct entries, %.1f s"
                  % (done, M, L, K, N, pool, elapsed),
    }
    out["torch_cpu"] = torch_cpu_comparator(w, entries)
    out["config1_cpu"] = config1_cpu()
    return out


def torch_cpu_comparator(w, entries, budget_s=6.0):
    """The reference's own CPU comparator (benchmark/pytorch/cpu/bmm_softmax_bmm.py:54-74): ``torch.bmm`` ->
    softmax -> ``torch.bmm`` in fp32 on the host cores, on the same single-batch entries as the port above."""
    import torch

    M, N, K, L = w["M"], w["N"], w["K"], w["L"]
    ts = [tuple(torch.from_numpy(x) for x in e) for e in entries[:8]]

    def run(q, k, v):
        s = torch.bmm(q, k)
        if w["kind"] == "softmax":
            s = torch.softmax(s * w["scale"], dim=2)
        return torch.bmm(s, v)

    run(*ts[0])
    done, elapsed = 0, 0.0
    while elapsed < budget_s and done < 100000:
        t0 = time.perf_counter()
        run(*ts[(done + 1) % len(ts)])
        elapsed += time.perf_counter() - t0
        done += 1
    return {"value": 2.0 * M * L * (K + N) * done / elapsed / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "sample": "%d single-batch-entry calls of torch.bmm / softmax / torch.bmm in fp32, %.1f s" % (done, elapsed)}


def config1_cpu(repeats=40):
    """The CPU-sized configuration exactly (fp32, batch 1, A[512x64].B[64x64].D[64x64], N(0,1), seed 0) through
    the fused CPU loop nest, one call per repeat with the caches flushed in between by streaming a buffer
    larger than the last-level cache (the protocol of benchmark/chimera/cpu/bmm_bmm_cpu.py:264-269,
    ``f_preproc="cache_flush_cpu_non_first_arg"``)."""
    import numpy as np

    from oracle import oracle as orc

    rng = np.random.default_rng(0)
    A = rng.standard_normal((1, 512, 64), dtype=np.float32)
    B = rng.standard_normal((1, 64, 64), dtype=np.float32)
    D = rng.standard_normal((1, 64, 64), dtype=np.float32)
    out = np.empty((1, 512, 64), dtype=np.float32)
    flush = np.zeros(1 << 27, dtype=np.uint8)  # 128 MiB streamed between calls
    orc.bmm_chain_fused_f32(A, B, D, inter="cast", out=out)
    cold, warm = [], []
    for i in range(repeats):
        flush += 1
        t0 = time.perf_counter()
        orc.bmm_chain_fused_f32(A, B, D, inter="cast", out=out)
        cold.append(time.perf_counter() - t0)
        t0 = time.perf_counter()
        orc.bmm_chain_fused_f32(A, B, D, inter="cast", out=out)
        warm.append(time.perf_counter() - t0)
    fl = 2.0 * 512 * 64 * (64 + 64)
    mean = sum(cold) / len(cold)
    return {"us_per_call": mean * 1e6, "gflops": fl / mean / 1e9, "us_per_call_caches_warm": min(warm) * 1e6,
            "cores": orc.num_threads(),
            "sample": "%d calls of the fp32 GEMM chain 512x64.64x64.64x64 through the fused CPU loop nest, "
                      "128 MiB streamed between calls" % repeats}


def run_one(name, steps, warmup, dev, long_run=False, zero_leg=True):
    w = WORKLOADS[name]
    wall_ms, ev_ms, gr_ms, tile, long_ms = time_gpu(w, steps, warmup, dev, long_run=long_run)
    fl, by = flops_of(w), bytes_of(w)
    short = SHORT[w["dtype"]]
    # The roofline uses the HIP-event time per launch of the eager loop (what rocprofv3's per-kernel
    # average agrees with); the graph replay of the same loop is reported beside it.
    k_ms = ev_ms
    tflops = fl / (k_ms * 1e-3) / 1e12
    if w["bound"] == "mfma":
        roof = {"bound": "mfma", "achieved": tflops, "peak": PEAK_TFLOPS[short], "unit": "TFLOP/s",
                "frac": tflops / PEAK_TFLOPS[short]}
    else:
        gbs = by / (k_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS}
    roof["traffic"] = measured_traffic(name, tile["variant"])
    roof["algorithmic_flops"] = fl
    roof["algorithmic_bytes"] = by
    roof["kernel_ms"] = k_ms
    roof["graph_replay_ms"] = gr_ms
    if long_ms is not None:
        roof["min_repeat_600ms_ms"] = long_ms
    if long_run and zero_leg and w["bound"] == "mfma" and w["kind"] in ("softmax", "cast"):
        # The same launch on all-zero operands: the same instruction stream without the switching activity of
        # real data.  The gap to kernel_ms is what the device's power management takes on N(0,1) operands.
        zcall, _ = make_call(w, dev, zero=True)
        warm_up(zcall, warmup)
        roof["zero_operand_kernel_ms"] = min_repeat_ms(zcall, 200.0)
    if w["kind"] == "conv" and w.get("groups", 1) == 1:
        # the same step with the weight repacking done once beforehand (ditto_conv_chain_prepare +
        # ditto_conv_chain_run_prepared): what a caller with fixed weights pays per call
        _, pev_ms, pgr_ms, _, _ = time_gpu(w, steps, warmup, dev, prepared=True)
        roof["weights_prepared_ms"] = pev_ms
        roof["weights_prepared_graph_replay_ms"] = pgr_ms
    return w, wall_ms, ev_ms, tile, roof


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-also", action="store_true", help="skip the brief runs of the other configurations")
    ap.add_argument("--no-zero", action="store_true",
                    help="skip the launches on all-zero operands (a kernel trace of the run then averages the launches on "
                         "N(0,1) operands only)")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MIB",
                    help="also launch one plain device copy of MIB MiB (read MIB, write MIB): a dispatch of known "
                         "traffic against which rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the chains shard over batch entries with no "
                 "exchange step, each GPU would run this same kernel on its share); --gpus %d is not supported" % args.gpus)

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.copy_probe > 0:
        src = torch.ones(args.copy_probe << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    w, wall_ms, ev_ms, tile, roof = run_one(args.workload, args.steps, args.warmup, dev, long_run=True,
                                            zero_leg=not args.no_zero)
    fl = flops_of(w)
    value = fl / (wall_ms * 1e-3) / 1e12
    short = SHORT[w["dtype"]]
    line = {
        "metric": "fused_chain_tflops",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "us_per_call": ev_ms * 1e3,
        "pct_of_mfma_peak": 100.0 * (fl / (ev_ms * 1e-3) / 1e12) / PEAK_TFLOPS[short],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": short,
        "data": "synthetic",
        "config": dict({"workload": args.workload, "description": w["desc"], "tile": tile},
                       **{k: v for k, v in w.items() if k not in ("kind", "dtype", "desc", "bound", "scale")}),
        "roofline": roof,
    }
    if not args.no_cpu and w["kind"] in ("softmax", "cast", "relu"):
        line["cpu_baseline"] = cpu_baseline(w)
    if not args.no_also:
        also = {}
        for name in WORKLOADS:
            if name == args.workload:
                continue
            ow, owall, oev, otile, oroof = run_one(name, 200, 20, dev)
            also[name] = {"us_per_call": oev * 1e3, "kernel_us": oroof["kernel_ms"] * 1e3,
                          "tflops": flops_of(ow) / (oroof["kernel_ms"] * 1e-3) / 1e12,
                          "roofline": {k: oroof[k] for k in ("bound", "achieved", "peak", "unit", "frac")}}
        line["also"] = also
    print(json.dumps(line))


if __name__ == "__main__":
    main()
