"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

TORCH_DTYPES = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32}


def to_dev(x, dtype, dev="cuda:0"):
    """fp32 numpy array (already rounded to ``dtype``) -> device tensor of that dtype (exact)."""
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev).to(TORCH_DTYPES[dtype])


def errors(got, want):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    d = got - want
    return float(np.abs(d).max()), float(np.linalg.norm(d) / max(np.linalg.norm(want), 1e-30))


def report(name, mx, rel):
    """Print the measured errors of a parity case (``pytest -s`` shows them; the figures recorded for
    the full-size configurations come from these lines)."""
    print("PARITY %s: max-abs %.3e rel-L2 %.3e" % (name, mx, rel), flush=True)
