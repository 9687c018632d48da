"""ctypes binding of ``libditto_chain_cpu.so``, the CPU target of the GEMM chain (``csrc/cpu/chain_cpu.cpp``).

A library of its own, loaded only when a chain is built for the ``llvm`` target: the HIP path never touches it.
The micro-kernel sources that ``auto_tensorize.cpu_intrin`` generates are compiled here with the host C compiler
into small shared objects (the reference compiles its generated kernels with clang and reaches them through
``call_extern``, python/ditto/auto_tensorize/intrinsic.py:601-603, 646-674).
"""
import ctypes
import hashlib
import os
import shutil
import subprocess
import tempfile
import threading

ABI_VERSION = 1
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libditto_chain_cpu.so")


class CpuChainDesc(ctypes.Structure):
    _fields_ = [
        ("abi_version", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("inter_op", ctypes.c_int32),
        ("relu_out", ctypes.c_int32),
        ("batch", ctypes.c_int64), ("M", ctypes.c_int64), ("N", ctypes.c_int64), ("K", ctypes.c_int64),
        ("L", ctypes.c_int64),
        ("a_batch_stride", ctypes.c_int64), ("a_row_stride", ctypes.c_int64),
        ("b_batch_stride", ctypes.c_int64), ("b_row_stride", ctypes.c_int64),
        ("c_batch_stride", ctypes.c_int64), ("c_row_stride", ctypes.c_int64),
        ("f_batch_stride", ctypes.c_int64), ("f_row_stride", ctypes.c_int64),
        ("softmax_scale", ctypes.c_float),
        ("mi", ctypes.c_int32), ("ni1", ctypes.c_int32), ("ni2", ctypes.c_int32),
        ("m_block", ctypes.c_int32), ("l_block", ctypes.c_int32), ("threads", ctypes.c_int32),
        ("update1", ctypes.c_void_p), ("update2", ctypes.c_void_p),
    ]


class CpuChainLibraryError(RuntimeError):
    pass


_lock = threading.Lock()
_lib = None
_kernels = {}  # source hash -> CDLL (kept alive: the nest calls into them)


def load():
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise CpuChainLibraryError("%s not found: build it with `python -m ditto_amd.build_ext` (needs g++)" % LIB_PATH)
            lib = ctypes.CDLL(LIB_PATH)
            lib.ditto_cpu_chain_abi_version.restype = ctypes.c_int
            lib.ditto_cpu_last_error.restype = ctypes.c_char_p
            lib.ditto_cpu_bmm_chain_run.restype = ctypes.c_int
            lib.ditto_cpu_bmm_chain_run.argtypes = [ctypes.POINTER(CpuChainDesc)] + [ctypes.c_void_p] * 4
            if lib.ditto_cpu_chain_abi_version() != ABI_VERSION:
                raise CpuChainLibraryError("libditto_chain_cpu.so has another ABI version than this binding")
            _lib = lib
    return _lib


def compile_kernel(source, symbol):
    """Compile a generated micro-kernel source and return the address of ``symbol`` (an ``<prefix>_update``
    function).  Objects are cached by source text for the life of the process."""
    key = hashlib.sha256(source.encode()).hexdigest()[:24]
    with _lock:
        lib = _kernels.get(key)
        if lib is None:
            cc = shutil.which("gcc") or shutil.which("cc")
            if not cc:
                raise CpuChainLibraryError("no C compiler for the generated micro-kernels")
            d = tempfile.mkdtemp(prefix="ditto_cpu_kernels_")
            src, so = os.path.join(d, key + ".c"), os.path.join(d, key + ".so")
            with open(src, "w") as f:
                f.write(source)
            r = subprocess.run([cc, "-O3", "-mavx2", "-mfma", "-fPIC", "-shared", "-o", so, src], capture_output=True,
                               text=True)
            if r.returncode != 0:
                raise CpuChainLibraryError("compiling the generated micro-kernel failed:\n%s" % r.stderr)
            lib = _kernels[key] = ctypes.CDLL(so)
    return ctypes.cast(getattr(lib, symbol), ctypes.c_void_p).value
