"""Build the gfx950 chain library (`libditto_chain.so`) in-tree with hipcc.

Usage: ``python -m ditto_amd.build_ext`` (or ``__graft_entry__.build()``).  Objects are
compiled in parallel, one hipcc process per translation unit, then linked into
``ditto_amd/csrc/libditto_chain.so``.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB = os.path.join(CSRC, "libditto_chain.so")
OBJ_DIR = os.path.join(CSRC, "build")
# the CPU target of the GEMM chain (build(..., target="llvm")): a library of its own, built with g++
CPU_LIB = os.path.join(CSRC, "libditto_chain_cpu.so")
CPU_SRC = os.path.join(CSRC, "cpu", "chain_cpu.cpp")
CPU_FLAGS = ["-O3", "-std=c++17", "-mavx2", "-mfma", "-fopenmp", "-fPIC", "-fvisibility=hidden", "-shared"]

# -packed-fp32-ops is switched off: packed fp32 VALU forms are not wanted in these kernels.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # let MFMA read and write its accumulator in arch VGPRs where the allocator can: the
    # inter-path op works on the accumulator, so AGPR-resident results cost a copy per use
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",
]

# The row maximum of the online softmax is only a stabiliser: without NaN-quieting the compiler
# need not canonicalise every MFMA result before v_max (one instruction saved per value).
FP_CHAIN_FLAGS = ["-fno-honor-nans"]

# (object name, source, extra defines)
UNITS = [
    ("api", "api.hip", []),
    ("gemm_chain_i8", "gemm_chain_i8.hip", []),
    ("gemm_chain_f32", "gemm_chain_f32.hip", []),
    ("conv_f16", "conv_chain_inst.hip", ["-DDITTO_INST_T=f16", "-DDITTO_INST_NAME=launch_conv_f16", "-DDITTO_PACK_NAME=pack_conv_w1_f16",
                                          "-DDITTO_INST2_NAME=launch_conv2_f16", "-DDITTO_PACK2_NAME=pack_conv_w2_f16", "-DDITTO_DW_NAME=launch_dw_conv_f16",
                                          "-DDITTO_RES_NAME=launch_conv_resident_f16", "-DDITTO_PACKRES_NAME=pack_conv_w2_resident_f16"]),
    ("conv_bf16", "conv_chain_inst.hip", ["-DDITTO_INST_T=bf16", "-DDITTO_INST_NAME=launch_conv_bf16", "-DDITTO_PACK_NAME=pack_conv_w1_bf16",
                                            "-DDITTO_INST2_NAME=launch_conv2_bf16", "-DDITTO_PACK2_NAME=pack_conv_w2_bf16", "-DDITTO_DW_NAME=launch_dw_conv_bf16",
                                            "-DDITTO_RES_NAME=launch_conv_resident_bf16", "-DDITTO_PACKRES_NAME=pack_conv_w2_resident_bf16"]),
    ("conv_rows_f16", "conv_rows_inst.hip", ["-DDITTO_INST_T=f16", "-DDITTO_CONVROWS_NAME=launch_conv_rows_f16"]),
    ("conv_rows_bf16", "conv_rows_inst.hip", ["-DDITTO_INST_T=bf16", "-DDITTO_CONVROWS_NAME=launch_conv_rows_bf16"]),
    ("dw_rows_f16", "dw_rows_inst.hip", ["-DDITTO_INST_T=f16", "-DDITTO_DWROWS_NAME=launch_dw_rows_f16"]),
    ("dw_rows_bf16", "dw_rows_inst.hip", ["-DDITTO_INST_T=bf16", "-DDITTO_DWROWS_NAME=launch_dw_rows_bf16"]),
    ("dw16_rows_f16", "dw16_rows_inst.hip", ["-DDITTO_INST_T=f16", "-DDITTO_DW16ROWS_NAME=launch_dw16_rows_f16"]),
    ("dw16_rows_bf16", "dw16_rows_inst.hip", ["-DDITTO_INST_T=bf16", "-DDITTO_DW16ROWS_NAME=launch_dw16_rows_bf16"]),
    ("fp_f16_cast", "bmm_chain_fp_inst.hip",
     ["-DDITTO_INST_T=f16", "-DDITTO_INST_INTER=0", "-DDITTO_INST_NAME=launch_f16_cast", *FP_CHAIN_FLAGS]),
    ("fp_f16_softmax", "bmm_chain_fp_inst.hip",
     ["-DDITTO_INST_T=f16", "-DDITTO_INST_INTER=2", "-DDITTO_INST_NAME=launch_f16_softmax", *FP_CHAIN_FLAGS]),
    ("fp_bf16_cast", "bmm_chain_fp_inst.hip",
     ["-DDITTO_INST_T=bf16", "-DDITTO_INST_INTER=0", "-DDITTO_INST_NAME=launch_bf16_cast", *FP_CHAIN_FLAGS]),
    ("fp_bf16_softmax", "bmm_chain_fp_inst.hip",
     ["-DDITTO_INST_T=bf16", "-DDITTO_INST_INTER=2", "-DDITTO_INST_NAME=launch_bf16_softmax", *FP_CHAIN_FLAGS]),
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the chain library needs ROCm to build")
    return exe


def _compile(unit):
    name, src, defs = unit
    obj = os.path.join(OBJ_DIR, name + ".o")
    extra = os.environ.get("DITTO_HIPCC_EXTRA", "").split()  # e.g. -D switches for experiments
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, *defs, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, " ".join(cmd), r.stderr))
    return obj


def build_cpu(verbose=True):
    """The CPU target's library (host code only)."""
    cxx = shutil.which("g++") or shutil.which("c++")
    if not cxx:
        raise RuntimeError("g++ not found; the CPU target of the chain needs a host C++ compiler")
    r = subprocess.run([cxx, *CPU_FLAGS, "-o", CPU_LIB, CPU_SRC], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building %s failed:\n%s" % (CPU_SRC, r.stderr))
    if verbose:
        print("built", CPU_LIB)
    return CPU_LIB


def build(verbose=True, jobs=None):
    """Compile every translation unit and link the shared library.  Always rebuilds."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    build_cpu(verbose)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, UNITS))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s" % r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
