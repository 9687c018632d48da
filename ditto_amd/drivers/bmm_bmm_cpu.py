"""GEMM -> GEMM chain on the CPU target (reference: benchmark/chimera/cpu/bmm_bmm_cpu.py).

The reference's flow, name for name: micro-kernel intrinsics from ``at.cpu_intrin``, the serial fusion state and
its tensorize axes, ``at.build_fusion_choice``, the hyper-fusion state, ``at.build_fusion_context`` with a CPU
hardware record, then for the first ``R`` ranked candidates ``fusionContext.run`` -> ``build(..., "llvm")`` ->
``time_evaluator`` with the cache flushed between runs, and the best time as a fraction of the server's peak.
Shapes are rounded up to the micro-kernel tile as the reference does (``uround``: M to 6, N and L to 16).
"""
import argparse
import os
import time

import numpy as np

import ditto_amd as ditto
from ditto_amd import auto_compute as ac
from ditto_amd import auto_tensorize as at
from ditto_amd.hardware import hardware_param

REPEAT = 20  # measurements per candidate (the reference takes 2000 runs of its compiled function)

# the reference's server records (bmm_bmm_cpu.py:27-53) and one for the machine at hand
ServerConfig = {
    "sc": dict(parallelism=20, cacheSizes=[32 * 16, 32 * 1024, 256 * 1024, 25344 * 1024], corePerLevel=[1.0, 1.0, 1.0, 10.0],
               bandwidth=[293.72, 81.72, 38.54, 13.14], isa="avx2", peakgflops=704.20),
    "sccc": dict(parallelism=32, cacheSizes=[32 * 16, 32 * 1024, 1024 * 1024, 25344 * 1024], corePerLevel=[1.0, 1.0, 1.0, 16.0],
                 bandwidth=[293.72, 81.72, 38.54, 13.14], isa="avx512", peakgflops=2150.50),
    "scccc": dict(parallelism=72, cacheSizes=[32 * 16, 32 * 1024 * 0.8, 1024 * 1024 * 0.8, 25344 * 1024 * 0.8],
                  corePerLevel=[1.0, 1.0, 1.0, 18.0], bandwidth=[293.72, 100.72, 50.54, 13.14], isa="avx512",
                  peakgflops=2995.20),
}


def local_server():
    """This machine: the cores this process may run on, AVX2 FMA peak at a nominal 2.5 GHz (2 x 8 lanes x 2 flops)."""
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    return dict(parallelism=cores, cacheSizes=[32 * 16, 32 * 1024, 1024 * 1024, 32 * 1024 * 1024],
                corePerLevel=[1.0, 1.0, 1.0, float(cores)], bandwidth=[293.72, 81.72, 38.54, 13.14], isa="avx2",
                peakgflops=cores * 2.5 * 32)


ServerConfig["local"] = local_server()


def ceil(x, y):
    return (x + y - 1) // y


def uround(x, y):
    return int(ceil(x, y) * y)


def tiles(K, L, N, isa):
    """(MI, NI1, KI1, NI2, KI2): the reference's setGlobals (:283-298) picks 6 x 16 tiles on AVX2 and 6 x 32 / 6 x 64 on
    AVX-512, with the first contraction's whole reduction (gcd(K, L) or 64) inside the intrinsic.  The chain builder of
    this package splits both reductions by one KI, so the intrinsic's reduction extent is 16 here; the micro-kernel
    takes the actual count at run time, so the generated code is the same."""
    del K, L
    if isa == "avx2":
        return 6, 16, 16, 16, 16
    ni = 64 if N % 64 == 0 else 32
    return 6, ni, 16, ni, 16


def test_double_gemm(batch, M, N, K, L, server, config=None):
    config = config or {}
    mode, dtype, verbose = config.get("mode", "survey"), config.get("dtype", "float32"), config.get("verbose", False)
    searchType = config.get("searchType", "stochastic")
    MI, NI1, KI1, NI2, KI2 = tiles(K, L, N, server["isa"])
    CPU = hardware_param(num_groups=server["parallelism"], cacheSizes=server["cacheSizes"], bandwidth=server["bandwidth"],
                         coresPerCacheLevel=server["corePerLevel"],
                         tensorWeight=config.get("tensorWeight", [1.0, 2.0, 1.0, 1.0, 1.0]), platform="CPU")
    ins, outs = ac.nn.functional.BatchGemmGemm(batch, M, N, K, L, dtype, dtype, MI=MI, NI=NI1, KI=KI2)
    assert NI1 == NI2 and KI1 == KI2
    t0 = time.time()
    layer = ac.layer([outs[0].op], inputs=ins)
    sfs = at.build_serial_fusion_state(layer)
    op1, op2 = sfs.first_op, sfs.second_op

    def get_match_info(op, shape, prefix):
        packed, code = at.cpu_intrin(op="gemm_noreshape", shape=shape, isa=server["isa"], dtype=dtype, prefix=prefix)
        choice = at.intrinsic_match(op.output(0), packed, ["SameRange"])[0]
        return at.match_info(choice, packed, code)

    first_match_info = get_match_info(op1, (MI, NI1, KI1), "gemm1")
    second_match_info = get_match_info(op2, (MI, NI2, KI2), "gemm2")
    sfs.register_tensorize_axes(list(first_match_info.axis) + list(second_match_info.axis))
    fuse_choice = at.build_fusion_choice(sfs, hw_param=CPU, dtype=dtype, simple_mode=-1)
    tensorize_state = at.tensorize_hyper_fusion_state(layer, fuse_choice, {op1: first_match_info, op2: second_match_info})
    fusionContext = at.build_fusion_context(sfs, layer, tensorize_state, "", hw_param=CPU, dtype=dtype,
                                            searchType=searchType, mode=mode)
    t1 = time.time()
    print("static analysis time", t1 - t0)
    rng = np.random.default_rng(0)
    inputs_np = [rng.uniform(-1, 1, [int(x) for x in y.shape]).astype(dtype) for y in ins]
    outputs_np = [np.zeros([int(x) for x in y.shape], dtype) for y in outs]
    want = (inputs_np[0].astype(np.float64) @ inputs_np[1].astype(np.float64)) @ inputs_np[2].astype(np.float64)
    R = 1 if mode == "test" else min(5, fusionContext.size)
    fusionLevel = fusionContext.getFusionLevel(0)
    top, top10 = 0.0, float("inf")
    for it in range(R):
        sch = fusionContext.run(it, None, verbose=verbose)
        func = ditto.build(sch, layer.schedule_tensors, "llvm", name="bmm")
        func(*inputs_np, *outputs_np)
        if not np.allclose(outputs_np[0], want, rtol=1e-3, atol=1e-3):
            print(f"WARNING: schedule {it} of {batch} {M} {N} {K} {L} is incorrect")
        evaluator = func.time_evaluator(func.entry_name, None, min_repeat_ms=0, repeat=REPEAT, number=1,
                                        f_preproc="cache_flush_cpu_non_first_arg")
        cost = evaluator(*inputs_np, *outputs_np).mean
        if it == 0:
            top = cost
        top10 = min(top10, cost)
        print(f"iter{it}: ", cost)
    return {"top1": top, "top10": top10}, fusionLevel, t1 - t0


def main(batch, M, N, K, L, dtype, server, mode):
    SERVER = ServerConfig[server]
    MI, NI1, _, NI2, _ = tiles(K, L, N, SERVER["isa"])
    B, M, N, L = batch, uround(M, MI), uround(N, NI2), uround(L, NI1)
    WORKLOAD = B * M * L * (K + N)
    print("B,M,N,K,L,dtype,WORKLOAD,SERVER")
    print(B, M, N, K, L, dtype, WORKLOAD, SERVER)
    t0 = time.time()
    Time, fusionLevel, _ = test_double_gemm(B, M, N, K, L, SERVER, config={"searchType": "normal", "verbose": False,
                                                                          "mode": mode, "dtype": dtype})
    t1 = time.time()
    print("schedule time: ", t1 - t0)
    ret = {}
    for k in Time:
        ret[k] = {"time(s)": Time[k], "%peak": (WORKLOAD / Time[k] / 1e9) / SERVER["peakgflops"]}
    ret["total_time"] = t1 - t0
    ret["fusionLevel"] = fusionLevel
    print(batch, M, N, K, L, dtype, ":", ret)
    return ret


example_text = "python -m ditto_amd.drivers.bmm_bmm_cpu --server local "

shapes = [
    # (batch, M, N, K, L)
    (8, 512, 512 // 8, 512 // 8, 512),      # Bert-Small
    (12, 512, 768 // 12, 768 // 12, 512),   # Bert-Base
    (16, 512, 1024 // 16, 1024 // 16, 512),  # Bert-Large
    (12, 256, 768 // 12, 768 // 12, 256),   # ViT-Base/14
    (16, 256, 1024 // 16, 1024 // 16, 256),  # ViT-Large/14
    (16, 256, 1280 // 16, 1280 // 16, 256),  # ViT-Huge/14
    (12, uround(196, 16), 768 // 12, 768 // 12, uround(196, 16)),   # ViT-Base/16
    (16, uround(196, 16), 1024 // 16, 1024 // 16, uround(196, 16)),  # ViT-Large/16
    (16, uround(196, 16), 1280 // 16, 1280 // 16, uround(196, 16)),  # ViT-Huge/16
    (1, 512, uround(49, 16), uround(49, 16), 256),  # Mixer-Small/32-S
    (1, 768, uround(49, 16), uround(49, 16), 384),  # Mixer-Base/32-S
    (1, 1024, uround(49, 16), uround(49, 16), 512),  # Mixer-Large/32-S
]

if __name__ == "__main__":
    parser = argparse.ArgumentParser(prog="base_maker", description="template maker", epilog=example_text,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--only_once", action="store_true")
    parser.add_argument("--dtype", type=str, choices=["float32", "float64"], default="float32")
    parser.add_argument("--begin", type=int, choices=list(range(len(shapes))), default=0)
    parser.add_argument("--num", type=int, choices=list(range(1, len(shapes) + 1)), default=len(shapes))
    parser.add_argument("--server", type=str, choices=sorted(ServerConfig), default="local")
    parser.add_argument("--mode", type=str, choices=["test", "best", "survey"], default="test")
    parser.add_argument("--store", type=int, choices=[0, 1], default=0)
    args = parser.parse_args()
    costs = []
    for ss in shapes[args.begin: args.begin + args.num]:
        B, M, N, K, L = ss
        costs.append((ss, main(batch=B, M=M, N=N, K=K, L=L, dtype=args.dtype, server=args.server, mode=args.mode)))
    print("B,M,N,K,L,dtype,args,sm,cost")
    for cc in costs:
        print(f"{cc[0]},{args.dtype},{args.server},{cc[1]}")
    for cc in costs:
        print(cc[1])
    if args.store:  # (the reference pickles the list; JSON here)
        import json

        with open("bmm_bmm_chimera.json", "w") as f:
            json.dump([[list(s), c] for s, c in costs], f)
