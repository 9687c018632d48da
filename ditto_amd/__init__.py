"""MI355X-native fused operator chains behind Ditto's hyper_fusion front-end.

    import ditto_amd as ditto
    from ditto_amd import auto_compute as ac, auto_tensorize as at, hardware as hw

The sub-packages keep the reference's names (``auto_compute``, ``auto_tensorize``,
``hardware``); ``ditto_amd.build`` stands where ``tvm.build`` is called on the scheduled
chain.  The compute runs in ``csrc/libditto_chain.so`` (hand-written gfx950 kernels behind the
C ABI of ``include/ditto_chain.h``); there is no CPU or PyTorch fallback for it.  The reference's CPU
target (``build(..., "llvm")`` on a schedule from ``tensorize_cpu`` / ``FusionContext.run``) is a path of
its own over host memory, ``csrc/libditto_chain_cpu.so``; neither target stands in for the other.  The
top-level package ``ditto`` re-exports these modules under the reference's import name.
"""
from . import auto_compute, auto_schedule, auto_tensorize, chimera, hardware, runtime, te  # noqa: F401
from .module import ChainFunction, build  # noqa: F401

__all__ = ["auto_compute", "auto_schedule", "auto_tensorize", "chimera", "hardware", "runtime", "te", "build",
           "ChainFunction"]
