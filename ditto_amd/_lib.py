"""ctypes binding of ``libditto_chain.so`` (the C ABI declared in ``include/ditto_chain.h``).

The library is loaded from ``ditto_amd/csrc``; there is no fallback implementation.
If it has not been built, loading raises ``RuntimeError`` telling how to build it.
"""
import ctypes
import os
import threading

ABI_VERSION = 2

# error codes (include/ditto_chain.h)
OK, EINVAL, EUNSUPPORTED, EHIP, EWORKSPACE = 0, -1, -2, -3, -4

# ditto_dtype
F16, BF16, F32, I8, I32, F64 = 0, 1, 2, 3, 4, 5
DTYPE_CODES = {"float16": F16, "bfloat16": BF16, "float32": F32, "int8": I8, "int32": I32, "float64": F64}
DTYPE_BYTES = {F16: 2, BF16: 2, F32: 4, I8: 1, I32: 4, F64: 8}

# ditto_inter_op
INTER_CAST, INTER_RELU, INTER_SOFTMAX, INTER_REQUANT = 0, 1, 2, 3
# ditto_b_layout
B_KL, B_LK = 0, 1


class BmmChainDesc(ctypes.Structure):
    _fields_ = [
        ("abi_version", ctypes.c_int32),
        ("in_dtype", ctypes.c_int32),
        ("acc_dtype", ctypes.c_int32),
        ("out_dtype", ctypes.c_int32),
        ("inter_op", ctypes.c_int32),
        ("b_layout", ctypes.c_int32),
        ("batch", ctypes.c_int64),
        ("M", ctypes.c_int64),
        ("N", ctypes.c_int64),
        ("K", ctypes.c_int64),
        ("L", ctypes.c_int64),
        ("a_batch_stride", ctypes.c_int64),
        ("a_row_stride", ctypes.c_int64),
        ("b_batch_stride", ctypes.c_int64),
        ("b_row_stride", ctypes.c_int64),
        ("c_batch_stride", ctypes.c_int64),
        ("c_row_stride", ctypes.c_int64),
        ("f_batch_stride", ctypes.c_int64),
        ("f_row_stride", ctypes.c_int64),
        ("softmax_scale", ctypes.c_float),
        ("requant_scale", ctypes.c_float),
        ("tile_variant", ctypes.c_int32),
        ("relu_out", ctypes.c_int32),
        ("batch_inner", ctypes.c_int64),
        ("a_batch_stride_outer", ctypes.c_int64),
        ("b_batch_stride_outer", ctypes.c_int64),
        ("c_batch_stride_outer", ctypes.c_int64),
        ("f_batch_stride_outer", ctypes.c_int64),
    ]


class ConvChainDesc(ctypes.Structure):
    _fields_ = [
        ("abi_version", ctypes.c_int32),
        ("in_dtype", ctypes.c_int32),
        ("acc_dtype", ctypes.c_int32),
        ("out_dtype", ctypes.c_int32),
        ("inter_op", ctypes.c_int32),
        ("relu_out", ctypes.c_int32),
        ("N", ctypes.c_int64),
        ("C0", ctypes.c_int64),
        ("H", ctypes.c_int64),
        ("W", ctypes.c_int64),
        ("C1", ctypes.c_int64),
        ("R1", ctypes.c_int64),
        ("S1", ctypes.c_int64),
        ("pad1", ctypes.c_int64),
        ("stride1", ctypes.c_int64),
        ("C2", ctypes.c_int64),
        ("R2", ctypes.c_int64),
        ("S2", ctypes.c_int64),
        ("pad2", ctypes.c_int64),
        ("stride2", ctypes.c_int64),
        ("groups1", ctypes.c_int64),
        ("tile_variant", ctypes.c_int32),
        ("reserved0", ctypes.c_int32),
    ]


class TileParam(ctypes.Structure):
    _fields_ = [
        ("block_threads", ctypes.c_int32),
        ("block_m", ctypes.c_int32),
        ("block_l", ctypes.c_int32),
        ("block_n", ctypes.c_int32),
        ("head_pad", ctypes.c_int32),
        ("lds_bytes", ctypes.c_int32),
        ("grid_x", ctypes.c_int32),
        ("grid_y", ctypes.c_int32),
        ("grid_z", ctypes.c_int32),
        ("variant", ctypes.c_int32),
    ]

    def to_json(self):
        return {name: getattr(self, name) for name, _ in self._fields_}


# Every symbol include/ditto_chain.h declares: (name, restype, argtypes)
_P = ctypes.c_void_p
EXPORTS = [
    ("ditto_chain_abi_version", ctypes.c_int, []),
    ("ditto_last_error", ctypes.c_char_p, []),
    ("ditto_bmm_chain_select_tile", ctypes.c_int, [ctypes.POINTER(BmmChainDesc), ctypes.POINTER(TileParam)]),
    ("ditto_conv_chain_select_tile", ctypes.c_int, [ctypes.POINTER(ConvChainDesc), ctypes.POINTER(TileParam)]),
    ("ditto_bmm_chain_workspace_bytes", ctypes.c_size_t, [ctypes.POINTER(BmmChainDesc)]),
    ("ditto_conv_chain_workspace_bytes", ctypes.c_size_t, [ctypes.POINTER(ConvChainDesc)]),
    ("ditto_bmm_chain_run", ctypes.c_int,
     [ctypes.POINTER(BmmChainDesc), _P, _P, _P, _P, _P, _P, ctypes.c_size_t, _P]),
    ("ditto_conv_chain_run", ctypes.c_int,
     [ctypes.POINTER(ConvChainDesc), _P, _P, _P, _P, _P, ctypes.c_size_t, _P]),
    ("ditto_conv_chain_prepare", ctypes.c_int,
     [ctypes.POINTER(ConvChainDesc), _P, _P, _P, ctypes.c_size_t, _P]),
    ("ditto_conv_chain_run_prepared", ctypes.c_int,
     [ctypes.POINTER(ConvChainDesc), _P, _P, _P, _P, _P, ctypes.c_size_t, _P]),
    ("ditto_conv_chain_run_static", ctypes.c_int, [ctypes.POINTER(ConvChainDesc), _P, _P, _P, _P, _P]),
]

STATIC_WORKSPACE_BYTES = 4 << 20  # DITTO_STATIC_WORKSPACE_BYTES

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libditto_chain.so")

_lock = threading.Lock()
_lib = None


class ChainLibraryError(RuntimeError):
    """The native chain library is missing or a call into it failed."""


def load():
    """Load (once) and return the ctypes handle of the chain library."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise ChainLibraryError(
                "%s not found: build it with `python -m ditto_amd.build_ext` (needs hipcc). "
                "There is no CPU or PyTorch fallback for the fused chains." % LIB_PATH
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, restype, argtypes in EXPORTS:
            fn = getattr(lib, name)  # AttributeError if the symbol is missing
            fn.restype = restype
            fn.argtypes = argtypes
        got = lib.ditto_chain_abi_version()
        if got != ABI_VERSION:
            raise ChainLibraryError("libditto_chain.so has ABI %d, binding expects %d" % (got, ABI_VERSION))
        _lib = lib
    return _lib


def last_error():
    return load().ditto_last_error().decode("utf-8", "replace")


def check(rc):
    """Map a C-ABI return code to the exceptions the reference raises at schedule time
    (descriptor errors -> ValueError, cf. TVMError from CHECK in hyper_fusion.cc:645-646)
    or at run time (HIP errors -> RuntimeError)."""
    if rc == OK:
        return
    msg = last_error()
    if rc in (EINVAL, EWORKSPACE):
        raise ValueError(msg)
    if rc == EUNSUPPORTED:
        raise NotImplementedError(msg)
    raise ChainLibraryError(msg)
