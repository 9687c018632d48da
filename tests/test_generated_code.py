"""Compiler-output checks (no GPU): the depthwise chain's register and address-space properties, and for every
kernel that no workgroup barrier is reached with the wave's own LDS accesses still in flight.

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


def barriers_with_lds_in_flight(asm_text):
    """[(kernel, instruction index)] of every ``s_barrier`` that some path through the kernel reaches while an LDS
    access of the same wave may still be outstanding.  A forward may-analysis over the kernel's control-flow graph:
    the state is the sequence of LDS (and scalar-load) instructions issued since the counter last read zero,
    ``s_waitcnt lgkmcnt(N)`` keeps the newest N of them, joins take the longer sequence."""
    import collections
    found = []
    cur, body = None, []
    kernels = []
    for line in asm_text.split("\n"):
        m = re.match(r"^(_Z\w+):", line)
        if m and "kernel" in m.group(1):
            cur, body = m.group(1), []
            continue
        if cur is not None:
            if line.startswith(".Lfunc_end"):
                kernels.append((cur, body))
                cur = None
            else:
                body.append(line)

    def join(a, b):
        if a is None:
            return b
        n = max(len(a), len(b))
        a, b = (0,) * (n - len(a)) + a, (0,) * (n - len(b)) + b
        return tuple(x | y for x, y in zip(a, b))

    for name, body in kernels:
        ins, labels = [], {}
        for raw in body:
            t = raw.strip()
            if not t or t.startswith(";"):
                continue
            m = re.match(r"^(\.LBB\w+):", t)
            if m:
                labels[m.group(1)] = len(ins)
                continue
            if t.startswith("."):
                continue
            ins.append(t.split(";")[0].strip())
        n = len(ins)
        succ = [[] for _ in range(n)]
        for i, t in enumerate(ins):
            op = t.split()[0]
            if op == "s_branch":
                succ[i].append(labels[t.split()[1]])
            elif op.startswith("s_cbranch"):
                succ[i].append(labels[t.split()[1]])
                if i + 1 < n:
                    succ[i].append(i + 1)
            elif op not in ("s_endpgm", "s_setpc_b64") and i + 1 < n:
                succ[i].append(i + 1)
        state = [None] * n
        state[0] = ()
        work = collections.deque([0])
        while work:
            i = work.popleft()
            s, t = state[i], ins[i]
            op = t.split()[0]
            if op.startswith("ds_"):
                s = (s + (1,))[-16:]
            elif op.startswith(("s_load", "s_buffer_load")):
                s = (s + (2,))[-16:]
            elif op == "s_waitcnt":
                m = re.search(r"lgkmcnt\((\d+)\)", t)
                if m:
                    keep = int(m.group(1))
                    s = s[len(s) - keep:] if keep < len(s) else s
                    if keep == 0:
                        s = ()
            for j in succ[i]:
                ns = join(state[j], s)
                if ns != state[j]:
                    state[j] = ns
                    work.append(j)
        found += [(name, i) for i, t in enumerate(ins) if t.startswith("s_barrier") and state[i] and 1 in
                  [k & 1 for k in state[i]]]
    return found


def _kernels(asm_text):
    """[(kernel symbol, [instruction text]), {label: instruction index}] per kernel of a device assembly listing."""
    out = []
    cur, body = None, []
    for line in asm_text.split("\n"):
        m = re.match(r"^(_Z\w+):", line)
        if m and "kernel" in m.group(1):
            cur, body = m.group(1), []
            continue
        if cur is not None:
            if line.startswith(".Lfunc_end"):
                ins, labels = [], {}
                for raw in body:
                    t = raw.strip()
                    if not t or t.startswith(";"):
                        continue
                    m = re.match(r"^(\.LBB\w+):", t)
                    if m:
                        labels[m.group(1)] = len(ins)
                        continue
                    if t.startswith("."):
                        continue
                    ins.append(t.split(";")[0].strip())
                out.append((cur, ins, labels))
                cur = None
            else:
                body.append(line)
    return out


def untracked_memory_ops_in_direct_load_loops(asm_text, loops_seen=None):
    """[(kernel, instruction)] of every memory instruction that shares a loop with a direct global -> LDS load
    (``buffer_load_dwordx4 ... lds``) and is not such a load itself.

    The BMM chain kernels issue those loads from inline asm and wait for them with hand-counted
    ``s_waitcnt vmcnt(N)``: "all but the newest N memory instructions of this wave have completed".  A spill
    store or reload (``scratch_*``), or any other global / buffer / flat access the compiler places inside the
    same loop, is one more memory instruction in that count: the wait then lets a tile be read before it has
    landed, silently.  Loops are the natural loops of the kernel's backward branches."""
    found = []
    for name, ins, labels in _kernels(asm_text):
        n = len(ins)
        succ = [[] for _ in range(n)]
        for i, t in enumerate(ins):
            op = t.split()[0]
            if op == "s_branch":
                succ[i].append(labels[t.split()[1]])
            elif op.startswith("s_cbranch"):
                succ[i].append(labels[t.split()[1]])
                if i + 1 < n:
                    succ[i].append(i + 1)
            elif op not in ("s_endpgm", "s_setpc_b64") and i + 1 < n:
                succ[i].append(i + 1)
        pred = [[] for _ in range(n)]
        for i in range(n):
            for j in succ[i]:
                pred[j].append(i)
        in_loop = set()
        for t in range(n):
            for h in succ[t]:
                if h <= t:  # a backward branch: its natural loop is everything that reaches t without passing h
                    body, stack = {h, t}, [t]
                    while stack:
                        x = stack.pop()
                        if x == h:
                            continue
                        for q in pred[x]:
                            if q not in body and q >= h:
                                body.add(q)
                                stack.append(q)
                    if any(re.match(r"buffer_load_dwordx4 .*\blds\b", ins[i]) for i in body):
                        in_loop |= body
                        if loops_seen is not None:
                            loops_seen.append((name, h, t))
        for i in sorted(in_loop):
            t = ins[i]
            if re.match(r"(scratch_|global_|flat_|buffer_)", t) and not re.match(r"buffer_load_dwordx4 .*\blds\b", t):
                found.append((name, t))
    return found


def test_direct_load_loop_analysis_on_a_small_kernel():
    clean = """
_Z6kernelv:
	scratch_store_dword off, v0, off
.LBB0_1:
	buffer_load_dwordx4 v1, s[0:3], 0 offen lds
	v_mfma_f32_16x16x32_bf16 v[0:3], v[4:7], v[8:11], v[0:3]
	s_waitcnt vmcnt(1)
	s_barrier
	s_cbranch_scc1 .LBB0_1
	scratch_load_dword v0, off, off
	global_store_dwordx4 v[2:3], v[4:7], off
	s_endpgm
.Lfunc_end0:
"""
    assert untracked_memory_ops_in_direct_load_loops(clean) == []
    # a reload the register allocator moved into the loop, and one in a cold block that branches back into it
    planted = clean.replace("	s_waitcnt vmcnt(1)", "	scratch_load_dword v9, off, off offset:4\n	s_waitcnt vmcnt(1)")
    assert untracked_memory_ops_in_direct_load_loops(planted) == [("_Z6kernelv", "scratch_load_dword v9, off, off offset:4")]
    cold = """
_Z6kernelv:
.LBB0_1:
	buffer_load_dwordx4 v1, s[0:3], 0 offen lds
	s_cbranch_vccnz .LBB0_3
.LBB0_2:
	s_waitcnt vmcnt(1)
	s_cbranch_scc1 .LBB0_1
	s_endpgm
.LBB0_3:
	global_load_dword v7, v[2:3], off
	s_branch .LBB0_2
.Lfunc_end0:
"""
    assert untracked_memory_ops_in_direct_load_loops(cold) == [("_Z6kernelv", "global_load_dword v7, v[2:3], off")]


@pytest.mark.parametrize("unit_name", ["fp_f16_cast", "fp_f16_softmax", "fp_bf16_cast", "fp_bf16_softmax"])
def test_bmm_chain_units_keep_their_counted_waits_exact(tmp_path, unit_name):
    """Every kernel of the four BMM chain units: no register spills at all, and no memory instruction other than
    the direct loads inside a loop that issues direct loads (see ``untracked_memory_ops_in_direct_load_loops``)."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    unit = [u for u in build_ext.UNITS if u[0] == unit_name][0]
    out = tmp_path / "unit.s"
    flags = [f for f in build_ext.HIPCC_FLAGS if f != "-fPIC"]
    cmd = [hipcc, *flags, "--cuda-device-only", "-S", *unit[2], os.path.join(CSRC, unit[1]), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    text = out.read_text()
    md = kernel_metadata(text)
    assert len(md) >= 14  # four-wave x {32, 64 rows} x 2 head sizes x 2 layouts, eight-wave, 16x16x32
    for name, v in md.items():
        assert v["vgpr_spill_count"] == 0, (name, v)
        # the eight-wave kernels and the 64-row kernel carry no scratch segment either (a kernel that has one starts
        # later, and the 64-row kernel runs launches of ten microseconds)
        if re.search(r"bmm_chain(8|8m16|4m16)_kernel", name):
            assert v["private_segment_fixed_size"] == 0, (name, v)
    loops = []
    assert untracked_memory_ops_in_direct_load_loops(text, loops) == []
    assert len({name for name, _, _ in loops}) == len(md)  # every kernel's tile loop was found and looked at
    assert barriers_with_lds_in_flight(text) == []


def test_barrier_analysis_on_a_small_kernel():
    text = """
_Z6kernelv:
	ds_write_b32 v0, v1
	s_cbranch_execz .LBB0_2
	ds_read_b32 v2, v0
	s_waitcnt lgkmcnt(0)
.LBB0_2:
	s_barrier
	ds_write_b32 v0, v1
	s_waitcnt lgkmcnt(0)
	s_barrier
	s_endpgm
.Lfunc_end0:
"""
    # the first barrier is reachable over the branch with the write still in flight, the second is not
    assert barriers_with_lds_in_flight(text) == [("_Z6kernelv", 4)]


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
    # every conv kernel of the unit: no barrier that a wave can reach with its own LDS accesses in flight (the
    # kernels wait explicitly in front of their barriers; a wave with all lanes masked off in the store blocks
    # used to reach the tile loop's barrier with its turn-around writes outstanding)
    assert barriers_with_lds_in_flight(text) == []


@pytest.mark.parametrize("unit_name", ["conv_rows_f16", "dw_rows_f16", "dw16_rows_f16"])
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
    # one instantiation per row width class (the kernel for sixteen outputs per channel: with and without ReLU;
    # the conv pipeline: 3x3 first and 1x1 first)
    assert len(md) == (8 if unit_name == "dw_rows_f16" else 16)
    for name, v in md.items():
        assert v["vgpr_spill_count"] == 0 and v["private_segment_fixed_size"] == 0, (name, v)
    lines = [l.strip() for l in text.split("\n") if l.strip() and not l.strip().startswith((";", "."))]
    barriers = [i for i, l in enumerate(lines) if l.startswith("s_barrier")]
    assert len(barriers) >= 8 * 2  # the loop barrier of each wave role
    for i in barriers:
        assert lines[i - 1].startswith("s_waitcnt lgkmcnt(0)"), lines[i - 3:i + 1]
    assert barriers_with_lds_in_flight(text) == []


@pytest.mark.parametrize("unit_name", ["gemm_chain_i8", "gemm_chain_f32"])
def test_no_barrier_with_lds_accesses_in_flight(tmp_path, unit_name):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    unit = [u for u in build_ext.UNITS if u[0] == unit_name][0]
    out = tmp_path / "unit.s"
    flags = [f for f in build_ext.HIPCC_FLAGS if f != "-fPIC"]
    cmd = [hipcc, *flags, "--cuda-device-only", "-S", *unit[2], os.path.join(CSRC, unit[1]), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    assert barriers_with_lds_in_flight(out.read_text()) == []
