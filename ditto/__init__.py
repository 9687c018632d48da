"""The reference's import name.  ``from ditto import auto_compute as ac``, ``import ditto.auto_tensorize as at``,
``from ditto.hardware.hw_param import hardware_param`` -- the first lines of the reference's drivers and tests --
resolve to the modules of ``ditto_amd`` (the same module objects, not copies), so such a script needs its
``import tvm`` / ``tvm.build`` lines changed and nothing else: ``ditto.build`` stands where ``tvm.build`` is called
on a scheduled chain."""
import importlib
import sys

import ditto_amd as _impl
from ditto_amd import ChainFunction, build  # noqa: F401

for _name in ("auto_compute", "auto_schedule", "auto_tensorize", "chimera", "hardware", "runtime", "te", "drivers"):
    globals()[_name] = importlib.import_module("ditto_amd." + _name)
for _full, _mod in list(sys.modules.items()):
    if _full.startswith("ditto_amd.") and not _full.split(".")[1].startswith("_"):
        sys.modules[__name__ + _full[len("ditto_amd"):]] = _mod
# the reference keeps its hardware record constructor in a module of its own (python/ditto/hardware/hw_param.py)
sys.modules[__name__ + ".hardware.hw_param"] = _impl.hardware

__all__ = list(_impl.__all__) + ["drivers"]
