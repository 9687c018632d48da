"""Hardware parameter tables (reference: python/ditto/hardware/hw_param.py:14-65,
python/ditto/hardware/__init__.py:18-54).  The chain path only ever treats the returned
object as an opaque argument of ``tensorize_cuda``; the MI355X entry is what the tile
table and the roofline report use.
"""
from dataclasses import dataclass, field
from typing import Sequence


@dataclass(frozen=True)
class HardwareParam:
    register_per_processor_kb: float = -1
    shared_memory_per_group_kb: float = -1
    shared_memory_bandwidth_gbs: float = -1
    global_memory_gb: float = -1
    global_memory_bandwidth_gbs: float = -1
    num_processors_per_group: int = -1
    num_groups: int = -1
    fp32_peak_perf_gflops: float = -1
    launch_latency_s: float = -1
    tensorWeight: Sequence[float] = (1.0, 1.0)
    cacheSizes: Sequence[float] = ()
    bandwidth: Sequence[float] = ()
    coresPerCacheLevel: Sequence[float] = ()
    platform: str = "NVGPU"
    # dense matrix-core peaks, GFLOP/s (GOP/s for int8); not in the reference's struct
    matrix_peak_gflops: dict = field(default_factory=dict)


def hardware_param(register_per_processor_kb=-1, shared_memory_per_group_kb=-1, shared_memory_bandwidth_gbs=-1,
                   global_memory_gb=-1, global_memory_bandwidth_gbs=-1, num_processors_per_group=-1,
                   num_groups=-1, fp32_peak_perf_gflops=-1, launch_latency_s=-1, tensorWeight=(1.0, 1.0),
                   cacheSizes=(), bandwidth=(), coresPerCacheLevel=(), platform="NVGPU", matrix_peak_gflops=None):
    return HardwareParam(register_per_processor_kb, shared_memory_per_group_kb, shared_memory_bandwidth_gbs,
                         global_memory_gb, global_memory_bandwidth_gbs, num_processors_per_group, num_groups,
                         fp32_peak_perf_gflops, launch_latency_s, tuple(float(x) for x in tensorWeight),
                         tuple(float(x) for x in cacheSizes), tuple(float(x) for x in bandwidth),
                         tuple(float(x) for x in coresPerCacheLevel), platform, dict(matrix_peak_gflops or {}))


# the reference's CUDA tables (python/ditto/hardware/devices/nvgpu/cuda_param.py)
_V100 = dict(register_per_processor_kb=64, shared_memory_per_group_kb=96, shared_memory_bandwidth_gbs=12080,
             global_memory_bandwidth_gbs=750, num_processors_per_group=4, num_groups=80,
             fp32_peak_perf_gflops=14e3, launch_latency_s=5e-6)
_A100 = dict(register_per_processor_kb=64, shared_memory_per_group_kb=164, shared_memory_bandwidth_gbs=12080,
             global_memory_bandwidth_gbs=1555, num_processors_per_group=4, num_groups=108,
             fp32_peak_perf_gflops=19.5e3, launch_latency_s=5e-6)
_CUDA = {
    "V100-16GB": hardware_param(global_memory_gb=16, **_V100),
    "V100-32GB": hardware_param(global_memory_gb=32, **_V100),
    "A100-40GB": hardware_param(global_memory_gb=40, **_A100),
    "A100-80GB": hardware_param(global_memory_gb=80, **_A100),
    "RTX3090": hardware_param(register_per_processor_kb=64, shared_memory_per_group_kb=128,
                              shared_memory_bandwidth_gbs=12080, global_memory_gb=24,
                              global_memory_bandwidth_gbs=760, num_processors_per_group=4, num_groups=68,
                              fp32_peak_perf_gflops=29.8e3, launch_latency_s=5e-6),
}
_CUDA["V100"] = _CUDA["V100-16GB"]
_CUDA["A100"] = _CUDA["A100-40GB"]

# AMD Instinct MI355X (gfx950, CDNA4): 256 CUs in 8 XCDs, 4 SIMDs per CU, 512 KB of vector
# registers and 160 KB of LDS per CU, 288 GB HBM3E at 8 TB/s; dense matrix peaks as published.
_HIP = {
    "MI355X": hardware_param(
        register_per_processor_kb=128, shared_memory_per_group_kb=160,
        shared_memory_bandwidth_gbs=256 * 256 * 2.4, global_memory_gb=288, global_memory_bandwidth_gbs=8000,
        num_processors_per_group=4, num_groups=256, fp32_peak_perf_gflops=157.3e3, launch_latency_s=5e-6,
        cacheSizes=(4 * 2 ** 20, 256 * 2 ** 20), platform="AMDGPU",
        matrix_peak_gflops={"float16": 2.5e6, "bfloat16": 2.5e6, "int8": 5.0e6, "float32": 157.3e3},
    )
}

QUERY_PARAM_FUNCS = {"gpu": {"cuda": lambda arch: _CUDA[arch.upper()], "hip": lambda arch: _HIP[arch.upper()]},
                     "cpu": {}}


def parse_target(target):
    """``device_type.programming_model.architecture``, e.g. ``gpu.cuda.A100`` or ``gpu.hip.MI355X``."""
    return target.split(".")


def query_hw_param(target):
    dev_type, pmodel, arch = parse_target(target)
    try:
        return QUERY_PARAM_FUNCS[dev_type][pmodel](arch)
    except KeyError:
        raise KeyError("unknown hardware target %r" % target)
