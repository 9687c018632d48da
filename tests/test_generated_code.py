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


@pytest.mark.parametrize("unit_name", ["conv_rows_f16", "dw_rows_f16"])
def test_row_kernels_use_no_scratch_and_wait_for_lds_before_every_barrier(tmp_path, unit_name):
    """The row kernels hand data between waves through LDS and count their outstanding loads by hand:

    * no scratch: a spill reload is a memory instruction the counted ``s_waitcnt vmcnt`` of the loading waves does
      not know of, and in the storing waves it would wait for every output store in flight;
    * every ``s_barrier`` directly behind ``s_waitcnt lgkmcnt(0)``: the compiler's own wait in front of a barrier
      was missing behind LDS writes under divergent control flow (a cold first launch then read three pixel slots
      before the write had landed), so the kernels spell the pair out."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    unit = [u for u in build_ext.UNITS if u[0] == unit_name][0]
    out = tmp_path / "rows.s"
    flags = [f for f in build_ext.HIPCC_FLAGS if f != "-fPIC"]
    cmd = [hipcc, *flags, "--cuda-device-only", "-S", *unit[2], os.path.join(CSRC, unit[1]), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    text = out.read_text()
    md = {k: v for k, v in kernel_metadata(text).items() if "rows_kernel" in k}
    assert len(md) == 8  # one instantiation per row width class
    for name, v in md.items():
        assert v["vgpr_spill_count"] == 0 and v["private_segment_fixed_size"] == 0, (name, v)
    lines = [l.strip() for l in text.split("\n") if l.strip() and not l.strip().startswith((";", "."))]
    barriers = [i for i, l in enumerate(lines) if l.startswith("s_barrier")]
    assert len(barriers) >= 8 * 3
    for i in barriers:
        assert lines[i - 1].startswith("s_waitcnt lgkmcnt(0)"), lines[i - 3:i + 1]
