"""Per-chain drivers: the counterparts of the reference's benchmark/chimera/cuda/*.py scripts
(same flags, shape tables, CSV header and cost unit).  Run as modules, e.g.
``python -m ditto_amd.drivers.bmm_softmax_bmm --in_dtype float16 --acc_dtype float32 --begin 0 --num 1``."""
