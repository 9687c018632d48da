"""Matrix-core contracts (reference: python/ditto/auto_tensorize/intrinsic.py:252-272 for
``cuda_wmma``, :37-48 for ``intrinsic_match``; src/auto_tensorize/intrinsic.cc:9-32).

``cuda_wmma`` keeps its signature; on this target it describes the same 16x16x16 logical
tile, which the gfx950 kernels execute with MFMA.  ``hip_mfma`` names the hardware tile
directly."""
from dataclasses import dataclass
from typing import List

from .. import te
from .pattern import IsCubic

# gfx950 dense MFMA tiles: (M, N, K) per input type
MFMA_SHAPES = {
    "float16": [(32, 32, 16), (16, 16, 32)],
    "bfloat16": [(32, 32, 16), (16, 16, 32)],
    "int8": [(32, 32, 32), (16, 16, 64)],
    "float32": [(32, 32, 2), (16, 16, 4)],
}
_ACC = {"float16": ("float32",), "bfloat16": ("float32",), "int8": ("int32",), "float32": ("float32",)}


@dataclass(frozen=True)
class TensorIntrin:
    name: str
    M: int
    N: int
    K: int
    in_dtype: str
    out_dtype: str
    scope: str = ""


@dataclass(frozen=True)
class PackedIntrinsic:
    load_intrinsics: tuple
    compute_intrinsic: TensorIntrin
    store_intrinsic: TensorIntrin
    load_scopes: tuple
    compute_scope: str
    store_scope: str

    def __str__(self):
        return "PackedIntrinsic(load=%s; compute=%s; store=%s)" % (
            [i.name for i in self.load_intrinsics], self.compute_intrinsic.name,
            self.store_intrinsic.name if self.store_intrinsic is not None else None)


def packed_intrinsic(loads, compute, store, load_scopes, compute_scope, store_scope):
    return PackedIntrinsic(tuple(loads), compute, store, tuple(load_scopes), compute_scope, store_scope)


def cuda_wmma(M=16, N=16, K=16, in_dtype="float16", out_dtype="float32", scope="global"):
    """The tensor-core contract of the reference: A/B tiles loaded row-major, accumulator
    fragment zero-filled, multiply-accumulated, stored row-major to ``scope``."""
    loads = [TensorIntrin("load_a", M, N, K, in_dtype, in_dtype, "shared"),
             TensorIntrin("load_b", M, N, K, in_dtype, in_dtype, "shared")]
    compute = TensorIntrin("gemm", M, N, K, in_dtype, out_dtype)
    store = TensorIntrin("store", M, N, K, out_dtype, out_dtype, scope)
    return packed_intrinsic(loads, compute, store, ["wmma.matrix_a", "wmma.matrix_b"], "wmma.accumulator",
                            "wmma.accumulator")


def hip_mfma(M=32, N=32, K=16, in_dtype="float16", out_dtype="float32", scope="vgpr"):
    """A gfx950 MFMA tile.  Operands come from VGPRs (loaded from LDS), the accumulator stays
    in VGPRs/AGPRs: ``scope`` is "vgpr" for the first contraction of a chain (its result is
    consumed in registers) and "global" for the second."""
    if in_dtype not in MFMA_SHAPES:
        raise ValueError("no MFMA for input type %s" % in_dtype)
    if (M, N, K) not in MFMA_SHAPES[in_dtype]:
        raise ValueError("no %dx%dx%d MFMA for %s; have %s" % (M, N, K, in_dtype, MFMA_SHAPES[in_dtype]))
    if out_dtype not in _ACC[in_dtype]:
        raise ValueError("MFMA on %s accumulates in %s, not %s" % (in_dtype, _ACC[in_dtype][0], out_dtype))
    loads = [TensorIntrin("lds_read_a", M, N, K, in_dtype, in_dtype, "lds"),
             TensorIntrin("lds_read_b", M, N, K, in_dtype, in_dtype, "lds")]
    compute = TensorIntrin("mfma_%dx%dx%d" % (M, N, K), M, N, K, in_dtype, out_dtype)
    store = TensorIntrin("store", M, N, K, out_dtype, out_dtype, scope)
    return packed_intrinsic(loads, compute, store, ["mfma.a", "mfma.b"], "mfma.accumulator", "mfma.accumulator")


def intrinsic_match(target: te.Tensor, packed_intrin: PackedIntrinsic, restrictions: List[str] = ()):
    """Iteration variables of ``target`` that map onto the intrinsic's (i, j, k).

    Returns a list of choices; callers take ``[0]`` = ``[mi, ni, rki]``
    (bmm_bmm_cuda.py:182-188).  With "InnerMost" the innermost spatial variable owned by each
    input and the innermost shared reduce variable are chosen; with "SameRange" their extents
    must equal the intrinsic's tile (for a 16^3 ``cuda_wmma`` tile; MFMA tiles are matched on
    divisibility, since the kernels re-tile the packed 16-blocks themselves).
    """
    op = target.op if isinstance(target, te.Tensor) else target
    if not IsCubic(op):
        return []
    intr = packed_intrin.compute_intrinsic
    n_in = len(op.accesses)

    def owned_by(i):
        return [iv for iv in op.axis
                if any(v is iv for v in op.accesses[i][1])
                and not any(any(v is iv for v in op.accesses[j][1]) for j in range(n_in) if j != i)]

    a_owned, b_owned = owned_by(0), owned_by(1)
    shared = [iv for iv in op.reduce_axis if all(any(v is iv for v in acc[1]) for acc in op.accesses)]
    if not a_owned or not b_owned or not shared:
        return []
    choices = []
    a_cands = a_owned[::-1] if "InnerMost" in restrictions else a_owned
    b_cands = b_owned[::-1] if "InnerMost" in restrictions else b_owned
    k_cands = shared[::-1] if "InnerMost" in restrictions else shared
    for mi in a_cands:
        for ni in b_cands:
            for ki in k_cands:
                if "SameRange" in restrictions:
                    is_mfma = intr.name.startswith("mfma_")  # wmma and CPU micro-kernel tiles match exactly
                    ok = ((mi.extent, ni.extent, ki.extent) == (intr.M, intr.N, intr.K)) if not is_mfma else (
                        mi.extent % 16 == 0 and ni.extent % 16 == 0 and ki.extent % 16 == 0)
                    if not ok:
                        continue
                choices.append([mi, ni, ki])
                if "InnerMost" in restrictions:
                    return choices
    return choices


def _cpu_gemm_source(name, M, N, K, dtype):
    """C source of the register-tile micro-kernel ``<name>_update``: ``c[M][N] += a[M][kc] . b[kc][N]`` on row-major
    tiles, the M x N accumulators held in ymm registers over the whole k loop (one broadcast of ``a`` per row and
    step against the vectors of a row of ``b``), and ``<name>_reset`` that clears a tile -- the two externs the
    reference's generated kernels export (intrinsic.py:292-416 for the 6 x 16 fp32 tile, :646-674 for the calls).
    ``K`` is the reduction extent the intrinsic was described with; the function takes the actual count."""
    fp32 = dtype == "float32"
    T, W = ("float", 8) if fp32 else ("double", 4)
    V, sfx = ("__m256", "ps") if fp32 else ("__m256d", "pd")
    bcast = "_mm256_broadcast_ss" if fp32 else "_mm256_broadcast_sd"
    nv, tail = N // W, N % W
    lines = ["#include <immintrin.h>",
             "/* %d x %d x %d %s register tile (%d vector accumulators%s) */" % (
                 M, N, K, dtype, M * nv, ", scalar tail of %d" % tail if tail else ""),
             "void %s_update(const %s* a, long lda, const %s* b, long ldb, %s* c, long ldc, long kc) {" % (name, T, T, T)]
    for r in range(M):
        for v in range(nv):
            lines.append("  %s acc%d_%d = _mm256_loadu_%s(c + %d * ldc + %d);" % (V, r, v, sfx, r, v * W))
    lines.append("  for (long k = 0; k < kc; ++k) {")
    for v in range(nv):
        lines.append("    const %s b%d = _mm256_loadu_%s(b + k * ldb + %d);" % (V, v, sfx, v * W))
    for r in range(M):
        lines.append("    { const %s av = %s(a + %d * lda + k);" % (V, bcast, r))
        for v in range(nv):
            lines.append("      acc%d_%d = _mm256_fmadd_%s(av, b%d, acc%d_%d);" % (r, v, sfx, v, r, v))
        lines.append("    }")
    if tail:
        lines.append("    for (int r = 0; r < %d; ++r) for (int j = %d; j < %d; ++j) c[r * ldc + j] += a[r * lda + k] * b[k * ldb + j];"
                     % (M, nv * W, N))
    lines.append("  }")
    for r in range(M):
        for v in range(nv):
            lines.append("  _mm256_storeu_%s(c + %d * ldc + %d, acc%d_%d);" % (sfx, r, v * W, r, v))
    lines.append("}")
    lines.append("void %s_reset(%s* c, long ldc) {" % (name, T))
    lines.append("  for (int r = 0; r < %d; ++r) for (int j = 0; j < %d; ++j) c[r * ldc + j] = 0;" % (M, N))
    lines.append("}")
    return "\n".join(lines) + "\n"


def cpu_intrin(op, shape, isa, dtype, prefix=""):
    """The CPU micro-kernel contract (reference: intrinsic.py:1675-1706): returns ``(packed_intrinsic, code)``.
    ``code`` is the C source of the register-tile kernel for that shape, exporting ``<prefix>_update`` and
    ``<prefix>_reset``; a chain built for the ``llvm`` target compiles it and runs its full tiles on it
    (``ditto_amd.build``).  AVX2 code is generated for either ``isa``; a tile wider than the sixteen ymm registers
    hold (more than twelve vector accumulators: the reference's 6 x 32 and 6 x 64 AVX-512 shapes) gets no code and
    is run by the nest in column panels of its own kernel.  The ``exp`` intrinsics carry no code: the nest applies
    the op between the contractions itself."""
    if op not in ("gemm", "gemm_noreshape", "conv", "exp", "exp_noreshape"):
        raise ValueError("unknown cpu intrinsic %r" % op)
    if isa not in ("avx2", "avx512"):
        raise ValueError("isa must be avx2 or avx512")
    if dtype not in ("float32", "float64"):
        raise ValueError("the CPU micro-kernels are fp32 / fp64 (intrinsic.py:283-291)")
    if op in ("exp", "exp_noreshape"):
        M, N = (int(x) for x in shape)
        K = 1
    else:
        M, N, K = (int(x) for x in shape[:3])
    name = prefix or op
    compute = TensorIntrin("%s_update" % name, M, N, K, dtype, dtype, "global")
    width = 8 if dtype == "float32" else 4
    fits = op in ("gemm", "gemm_noreshape") and 1 <= M <= 6 and M * (N // width) <= 12 and N >= width
    code = _cpu_gemm_source(name, M, N, K, dtype) if fits else ""
    return packed_intrinsic([], compute, None, ["global", "global"], "global", "global"), code
