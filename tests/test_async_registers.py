"""Compiler-output check for the persistent conv chain (no GPU): the halo tile of the next output tile
is fetched by inline-asm buffer loads that the compiler does not track, and consumed only after a
hand-placed ``s_waitcnt``.  That is safe only while nothing reads, copies or spills the destination
registers in between -- a register-allocator copy would take stale values, and the register freed by
it would later be overwritten by the returning load.  The test compiles the kernels to assembly and
verifies that the only instructions touching those registers are the byte permutes of the staging
step that follows the wait."""
import collections
import os
import re
import shutil
import subprocess

import pytest

from ditto_amd import build_ext

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ditto_amd", "csrc")


def _regs(text):
    s = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
        s |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bv(\d+)\b", text):
        s.add(int(m.group(1)))
    return s


def async_register_uses(asm_text):
    """{kernel: Counter(mnemonic -> count)} of compiler-emitted instructions that touch a register
    written by an inline-asm buffer load (direct-to-LDS loads have no register destination)."""
    lines = asm_text.split("\n")
    starts = [i for i, l in enumerate(lines) if re.match(r"^_ZN5ditto\S+:", l)]
    out = {}
    for k, start in enumerate(starts):
        body = lines[start:starts[k + 1] if k + 1 < len(starts) else len(lines)]
        in_asm, tracked, asm_lines = False, set(), set()
        for i, l in enumerate(body):
            if "#ASMSTART" in l:
                in_asm = True
            elif "#ASMEND" in l:
                in_asm = False
            elif in_asm:
                asm_lines.add(i)
                if "buffer_load_dwordx" in l and " lds" not in l:
                    tracked |= _regs(l.split()[1])
        if not tracked:
            continue
        uses = collections.Counter()
        for i, l in enumerate(body):
            if i in asm_lines or not l.startswith("\t") or l.strip().startswith(";"):
                continue
            if _regs(l) & tracked:
                uses[l.split()[0]] += 1
        out[body[0].split(":")[0]] = (len(tracked), uses)
    return out


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_async_halo_registers_are_only_read_after_the_wait(tmp_path, dtype):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    out = tmp_path / "persist.s"
    flags = [f for f in build_ext.HIPCC_FLAGS if f != "-fPIC"]
    cmd = [hipcc, *flags, "--cuda-device-only", "-S", "-DDITTO_INST_T=" + dtype,
           "-DDITTO_PERSIST_NAME=launch_conv_persist_" + dtype, os.path.join(CSRC, "conv_chain_persist_inst.hip"),
           "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    found = async_register_uses(out.read_text())
    assert len(found) == 8  # (C1 tiles 1 | 2) x (32 | 64 input channels) x (1x1 | 3x3 first filter)
    for name, (nregs, uses) in found.items():
        assert nregs == 32, name  # eight 16-byte loads per thread
        assert set(uses) == {"v_perm_b32"} and uses["v_perm_b32"] == 32, (name, dict(uses))
