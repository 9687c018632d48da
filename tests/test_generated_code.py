"""Compiler-output checks for the depthwise chain (no GPU).

Two properties of the generated code decide the speed of the persistent depthwise kernel and are
invisible in its results:

* no scratch in the variants with 16-byte output stores: a reload from scratch is followed by
  ``s_waitcnt vmcnt(0)``, which also waits for every output store still in flight -- with a reload at the
  top of the tile loop each tile waited for the previous tile's stores (83 us instead of 45 us on the
  32 x 32 x 112 x 112, multiplier 1 case);
* no flat memory instructions: a pointer that has passed through an ``asm`` constraint is no longer known
  to point to global memory or LDS, and flat accesses count on both wait counters.
"""
import os
import re
import shutil
import subprocess

import pytest

from ditto_amd import build_ext

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ditto_amd", "csrc")


def kernel_metadata(asm_text):
    """{kernel symbol: {"vgpr_spill_count": n, "private_segment_fixed_size": n}} from the code object notes."""
    out, name = {}, None
    for line in asm_text.split("\n"):
        m = re.match(r"\s+\.name:\s+(\S+)", line)
        if m:
            name = m.group(1)
            continue
        m = re.match(r"\s+\.(vgpr_spill_count|private_segment_fixed_size):\s+(\d+)", line)
        if m and name:
            out.setdefault(name, {})[m.group(1)] = int(m.group(2))
    return out


def test_kernel_metadata_parser():
    text = """
    .name:           _ZN5ditto1aEv
    .private_segment_fixed_size: 0
    .vgpr_spill_count: 0
    .name:           _ZN5ditto1bEv
    .private_segment_fixed_size: 112
    .vgpr_spill_count: 28
"""
    md = kernel_metadata(text)
    assert md["_ZN5ditto1aEv"] == {"private_segment_fixed_size": 0, "vgpr_spill_count": 0}
    assert md["_ZN5ditto1bEv"] == {"private_segment_fixed_size": 112, "vgpr_spill_count": 28}


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_depthwise_kernels_with_wide_stores_use_no_scratch_and_no_flat_accesses(tmp_path, dtype):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    unit = [u for u in build_ext.UNITS if u[0] == "conv_" + dtype][0]
    out = tmp_path / "conv.s"
    flags = [f for f in build_ext.HIPCC_FLAGS if f != "-fPIC"]
    cmd = [hipcc, *flags, "--cuda-device-only", "-S", *unit[2], os.path.join(CSRC, unit[1]), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    text = out.read_text()
    assert not re.search(r"\bflat_(load|store|atomic)", text)
    md = kernel_metadata(text)
    # template arguments <T, C2T, PXW, NG, WIDE, F33, MSH>: WIDE is the fifth
    wide = {k: v for k, v in md.items() if re.search(r"dw_conv_mfma_kernelI\S+?Li\d+ELi\d+ELi\d+ELb1ELb[01]E", k)}
    assert len(wide) >= 24  # 4 output widths x (3x3 | other filters | four vector-ALU multipliers)
    for name, v in wide.items():
        assert v["vgpr_spill_count"] == 0 and v["private_segment_fixed_size"] == 0, (name, v)
