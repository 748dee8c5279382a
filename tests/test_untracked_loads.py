"""The tiled GEMM loads its weight fragments into registers with loads the compiler does not know of (inline assembly,
completion tracked by hand with ``s_waitcnt vmcnt``): between the issue of such a load and the wait that covers it,
nothing may read or write its destination registers, and the compiler is free to break that by moving or copying a
register it believes to be ready.  This test compiles the kernel to device assembly and walks the K loops of the
fragment-ordered forms in the order they execute, three passes in a row, replaying the ``vmcnt`` bookkeeping of the
code itself; any instruction that touches a register while a load into it may be in flight fails the test.  It runs
on the CPU (hipcc cross-compiles) and is meant to be re-run after a compiler change."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def registers(text: str) -> set:
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", text):
        if m.group(1):
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def walk_loop(body, passes=3):
    """``body``: the instructions of a straight-line loop body.  Returns the violations of passes 2.. (the first pass
    only fills the queues of outstanding operations as the previous iteration would have left them).

    Operations of one kind (register loads, copies into LDS, stores) complete in order, operations of different kinds
    need not; one counter covers all.  ``s_waitcnt vmcnt(n)`` therefore proves an operation complete only if at least n
    operations of its own kind were issued after it: per kind, all but the last n are known to have landed."""
    queues = {"load": [], "copy": [], "store": []}   # per outstanding operation: its destination registers
    violations = []
    for it in range(passes):
        for line in body:
            op = line.split()[0]
            if op.startswith("s_waitcnt"):
                m = re.search(r"vmcnt\((\d+)\)", line)
                if m:
                    for q in queues.values():
                        del q[: max(0, len(q) - int(m.group(1)))]
                continue
            in_flight = set().union(*queues["load"]) if queues["load"] else set()
            used = registers(line.split(None, 1)[1]) if " " in line else set()
            if it > 0 and used & in_flight:
                violations.append((it, line, sorted(used & in_flight)[:4]))
            if op.startswith("global_load_lds"):
                queues["copy"].append(set())
            elif op.startswith(("global_store", "buffer_store")):
                queues["store"].append(set())
            elif op.startswith(("global_load", "buffer_load")):
                queues["load"].append(registers(line.split(None, 1)[1].split(",")[0]))
    return violations


def straight_line_loops(lines):
    labels = {l[:-1]: i for i, l in enumerate(lines) if l.endswith(":")}
    for i, l in enumerate(lines):
        if l.startswith(("s_cbranch", "s_branch")):
            target = l.split()[-1]
            if target in labels and labels[target] <= i:
                body = [x for x in lines[labels[target]:i] if not x.endswith(":") and not x.startswith(".")]
                if not any(x.startswith(("s_cbranch", "s_branch")) for x in body):
                    yield body


def test_the_walker_sees_a_register_touched_in_flight():
    ok = ["global_load_dwordx4 v[4:7], v1, s[2:3]", "s_waitcnt vmcnt(0)", "v_mfma_f32_32x32x16_bf16 a[0:15], v[4:7], v[8:11], a[0:15]"]
    assert walk_loop(ok) == []
    early = ["global_load_dwordx4 v[4:7], v1, s[2:3]", "v_mov_b32_e32 v9, v5", "s_waitcnt vmcnt(0)"]
    assert walk_loop(early)
    # a wait that leaves one operation outstanding covers the older of two loads only
    partly = ["global_load_dwordx4 v[4:7], v1, s[2:3]", "global_load_dwordx4 v[12:15], v1, s[2:3]", "s_waitcnt vmcnt(1)",
              "v_mov_b32_e32 v9, v5", "v_mov_b32_e32 v10, v13", "s_waitcnt vmcnt(0)"]
    assert [v[1] for v in walk_loop(partly, passes=2)] == ["v_mov_b32_e32 v10, v13"]
    # a copy into LDS issued after a register load proves nothing about that load
    mixed = ["global_load_dwordx4 v[4:7], v1, s[2:3]", "global_load_lds_dwordx4 v2, s[4:5]", "s_waitcnt vmcnt(1)",
             "v_mov_b32_e32 v9, v5", "s_waitcnt vmcnt(0)"]
    assert walk_loop(mixed, passes=2)


@pytest.mark.timeout(600)
def test_fragment_loads_of_the_tiled_gemm_stay_untouched_until_their_wait(tmp_path):
    from mase_amd import build

    if shutil.which(build.HIPCC) is None and not os.path.exists(build.HIPCC):
        pytest.skip("no hipcc")
    flags = [f for f in build.COMMON_FLAGS if f not in ("-Wall", "-Wno-unused-function")]
    out = tmp_path / "gemm_bf16.s"
    cmd = [build.HIPCC, *flags, "-I", os.path.join(ROOT, "mase_amd", "csrc"), "-I", os.path.join(ROOT, "include"),
           "-S", "--cuda-device-only", os.path.join(ROOT, "mase_amd", "csrc", "gemm_bf16.hip"), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    text = out.read_text()
    checked = 0
    for m in re.finditer(r"\n(_Z\w*gemm_bf16_tn_kernel\w*):[^\n]*\n(.*?)\.Lfunc_end", text, re.S):
        lines = [l.split(";")[0].strip() for l in m.group(2).split("\n")]
        lines = [l for l in lines if l]
        for body in straight_line_loops(lines):
            register_loads = [x for x in body if re.match(r"global_load_dword(x\d)? v", x)]
            if not register_loads or not any(x.startswith("v_mfma") for x in body):
                continue
            checked += 1
            violations = walk_loop(body)
            assert not violations, (m.group(1), violations[:5])
    # the K loops of the fragment-ordered forms (bf16 image and MXINT8 codes, three output types each)
    assert checked >= 6, checked
