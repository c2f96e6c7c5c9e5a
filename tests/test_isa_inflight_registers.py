"""The grouped GEMM kernels issue their global loads through inline assembly and wait for them by count (load16_async /
wait_loads / wait_vm in csrc/): between a request and the wait that covers it the destination register holds no data yet,
which the compiler does not know. A register allocator that splits such a variable's live range inside the K loop and
restores it with a copy (at a loop's back edge, say) makes the kernel read the register before the load has landed - the
results are then wrong now and then, and the late load hits whatever the register was reused for. Nothing in the source
can forbid that, so the generated code is checked: inside the K loops, a basic block that does not drain the load queue
(s_waitcnt vmcnt(0)) must not copy a register that some hand-issued load writes. Blocks on the drain path (past the last
K block, where every register is waited for before its next use) may.

CPU only: the device code is compiled to assembly with hipcc, nothing runs."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "flyingfish_amd", "csrc")
FLAGS = ["-x", "hip", "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument", "--cuda-device-only", "-S"]
COPIES = ("v_mov_b32_e32", "v_mov_b64_e32", "v_accvgpr_write_b32")


def _regs(tok):
    tok = tok.strip().rstrip(",")
    m = re.match(r"^v\[(\d+):(\d+)\]$", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"^v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def _kernels(text):
    lines = text.split("\n")
    starts = [(i, re.match(r"^(_ZN5ffmoe\w+):", l).group(1)) for i, l in enumerate(lines) if re.match(r"^_ZN5ffmoe\w+:", l)]
    for n, (i, name) in enumerate(starts):
        end = starts[n + 1][0] if n + 1 < len(starts) else len(lines)
        yield name, lines[i:end]


def _suspect_blocks(body):
    """(block, copies) for K-loop blocks without a full drain that copy registers written by hand-issued loads."""
    dests, inasm = set(), False
    for l in body:
        if "ASMSTART" in l:
            inasm = True
        elif "ASMEND" in l:
            inasm = False
        else:
            t = l.strip().replace(",", " ").split()
            if inasm and t and t[0].startswith("global_load"):
                dests |= _regs(t[1])
    if not dests:
        return None
    out, blk = [], None
    for l in body + [".LBB_end:"]:
        if l.startswith(".LBB") or l.startswith("; %bb"):
            if blk and blk["loop"] and not blk["drain"] and blk["wide"]:
                out.append((blk["name"], blk["wide"]))
            blk = {"name": l.split()[0] if l.startswith(".LBB") else l.split()[1], "loop": "Depth=2" in l or "Depth=3" in l, "drain": False, "wide": []}
            continue
        if blk is None:
            continue
        t = l.strip().replace(",", " ").split()
        if not t:
            continue
        if t[0] == "s_waitcnt" and "vmcnt(0)" in l:
            blk["drain"] = True
        # 64-bit copies are pieces of a 128-bit load destination on the move; single words are the per-set scales, which
        # the kernels copy on purpose once they have landed
        if t[0] == "v_mov_b64_e32" and len(t) >= 3 and _regs(t[2]) & dests:
            blk["wide"].append(l.strip())
    return out


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not on PATH")
def test_no_copy_of_a_register_with_a_load_in_flight(tmp_path):
    asm = tmp_path / "prefill.s"
    r = subprocess.run(["hipcc", *FLAGS, "-o", str(asm), os.path.join(CSRC, "prefill.hip")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    checked, bad = 0, []
    for name, body in _kernels(asm.read_text()):
        sus = _suspect_blocks(body)
        if sus is None:
            continue
        checked += 1
        for block, copies in sus:
            bad.append("%s %s: %s" % (name, block, "; ".join(copies[:3])))
    assert checked >= 20, "kernels with hand-issued loads found: %d" % checked
    assert not bad, "copies of load destinations outside a drain block:\n" + "\n".join(bad[:20])
