"""Static check of the hand-pipelined kernels (no GPU needed).

The expanded-table kernels issue LDS reads and global loads in inline assembly and wait for them with explicit
s_waitcnt blocks, so the compiler does not know that the destination registers of such an instruction are still being
written.  It is free to copy one of them (at a merge point of the control flow, or in front of an assembly block that
ties it as an in/out operand): a copy that sits between the load and its wait reads stale data.  This test compiles the
device code to assembly and walks every kernel: between an asynchronous load and the wait that covers it no instruction
may name one of its destination registers.  Likewise a 128-bit store written in assembly must be followed by two idle
cycles before its data registers are written again.
"""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "appmult-aware-retraining_amd"))
import build as amr_build  # noqa: E402

SOURCES = ["lutgemm_fwd_slab.hip", "lutgemm_gradA_slab.hip"]


def _vgprs(text):
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", text):
        if m.group(1):
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def scan(asm_text):
    """Returns [(kernel, line number, instruction, registers)] of instructions that touch a register in flight.

    Linear walk per kernel.  LDS reads complete in order: s_waitcnt lgkmcnt(n) leaves the n youngest in flight.  For
    vector-memory loads only the interval up to the next vmcnt wait is checked (the code between a load and its wait
    may have been laid out elsewhere in the file, so the count itself is not modelled)."""
    hits, kernel, lds, vmem = [], None, [], []
    for ln, raw in enumerate(asm_text.split("\n"), 1):
        t = raw.strip()
        m = re.match(r"^(_Z\w+):", t)
        if m:
            kernel, lds, vmem = m.group(1), [], []
            continue
        if kernel is None or not t or t[0] in ";.":
            continue
        t = t.split(";")[0].strip()
        if not t:
            continue
        op, args = t.split()[0], t[len(t.split()[0]):]
        if op == "s_endpgm":
            lds, vmem = [], []
            continue
        if op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", args)
            if m:
                lds = lds[len(lds) - int(m.group(1)):] if int(m.group(1)) else []
            if "vmcnt" in args:
                vmem = []
            continue
        if op.startswith("s_"):
            continue
        pending = set().union(*lds, *vmem) if (lds or vmem) else set()
        touched = _vgprs(args) & pending
        if touched:
            hits.append((kernel, ln, t, sorted(touched)))
        first = args.split(",")[0]
        if op.startswith("ds_read"):
            lds.append(_vgprs(first))
        elif op.startswith("ds_"):
            lds.append(set())
        elif op.startswith("global_load_lds"):
            pass
        elif op.startswith("global_load") or op.startswith("buffer_load") or op.startswith("scratch_load"):
            vmem.append(_vgprs(first))
    return hits


def scan_wide_stores(asm_text):
    """Returns [(line number, store, next instruction)]: a store of more than 64 bits written in an assembly block whose data
    registers are written within the two cycles that follow it.  The hardware still reads the data then; the compiler
    inserts the idle cycles after its own stores only."""
    hits, in_asm, watch = [], False, []          # watch: [data registers, cycles left, line, text]
    for ln, raw in enumerate(asm_text.split("\n"), 1):
        t = raw.strip()
        if "#ASMSTART" in t:
            in_asm = True
            continue
        if "#ASMEND" in t:
            in_asm = False
            continue
        if not t or t[0] in ";.":
            continue
        t = t.split(";")[0].strip()
        if not t or t.endswith(":"):
            continue
        op, args = t.split()[0], t[len(t.split()[0]):]
        if op == "s_nop":
            idle = int(args.strip(), 0) + 1
            watch = [[r, left - idle, l0, t0] for r, left, l0, t0 in watch if left - idle > 0]
            continue
        written = _vgprs(args.split(",")[0]) if op.startswith("v_") or "load" in op or op.startswith("ds_read") else set()
        for r, left, l0, t0 in watch:
            if r & written:
                hits.append((l0, t0, t))
        watch = [[r, left - 1, l0, t0] for r, left, l0, t0 in watch if left - 1 > 0]
        if in_asm and re.match(r"(global|flat|buffer|scratch)_store_dwordx[34]", op):
            watch.append([_vgprs(args.split(",")[1]), 2, ln, t])
    return hits


def test_scanner_sees_a_write_behind_a_wide_store():
    bad = """	;;#ASMSTART
	global_store_dwordx4 v[62:63], v[52:55], off
	;;#ASMEND
	v_readlane_b32 s7, v127, 7
	v_lshl_add_u64 v[52:53], v[62:63], 0, s[6:7]
"""
    assert [h[0] for h in scan_wide_stores(bad)] == [2]
    assert scan_wide_stores(bad.replace("off\n", "off\n s_nop 1\n")) == []
    assert scan_wide_stores(bad.replace("v[52:53], v[62:63]", "v[56:57], v[62:63]")) == []
    assert scan_wide_stores(bad.replace("dwordx4 v[62:63], v[52:55]", "dwordx2 v[62:63], v[52:53]")) == []


def test_scanner_sees_a_copy_in_front_of_the_wait():
    bad = """_Zkernel:
	ds_read_b128 v[4:7], v1
	v_mov_b64_e32 v[10:11], v[4:5]
	s_waitcnt lgkmcnt(0)
	v_add_f32_e32 v0, v4, v10
	s_endpgm
"""
    good = bad.replace("	v_mov_b64_e32 v[10:11], v[4:5]\n	s_waitcnt lgkmcnt(0)\n", "	s_waitcnt lgkmcnt(0)\n	v_mov_b64_e32 v[10:11], v[4:5]\n")
    assert [h[1] for h in scan(bad)] == [3]
    assert scan(good) == []
    # in-order completion: with two reads in flight lgkmcnt(1) covers the older one only
    two = """_Zkernel:
	ds_read_b64 v[2:3], v1
	ds_read_b64 v[4:5], v1 offset:8
	s_waitcnt lgkmcnt(1)
	v_mov_b32_e32 v8, v2
	v_mov_b32_e32 v9, v4
	s_endpgm
"""
    assert [h[1] for h in scan(two)] == [6]
    vm = """_Zkernel:
	global_load_dword v34, v[20:21], off
	v_lshrrev_b32_e32 v0, 8, v34
	s_waitcnt vmcnt(0)
	v_lshrrev_b32_e32 v0, 8, v34
	s_endpgm
"""
    assert [h[1] for h in scan(vm)] == [3]


@pytest.mark.parametrize("source", SOURCES)
def test_no_instruction_touches_a_register_whose_load_is_in_flight(source, tmp_path):
    out = tmp_path / (source + ".s")
    cmd = ["hipcc"] + amr_build.FLAGS + ["--cuda-device-only", "-S", os.path.join(amr_build.CSRC, source), "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    hits = scan(out.read_text())
    assert not hits, "\n".join(f"{k}: line {ln}: {ins}  <- in flight: {regs}" for k, ln, ins, regs in hits[:20])
    wide = scan_wide_stores(out.read_text())
    assert not wide, "\n".join(f"line {ln}: {st}  <- data written by: {ins}" for ln, st, ins in wide[:20])
