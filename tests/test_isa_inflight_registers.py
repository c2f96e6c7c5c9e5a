"""The grouped GEMM kernels issue their global loads through inline assembly and wait for them by count (load16_async /
wait_loads / wait_vm in csrc/): between a request and the wait that covers it the destination register holds no data yet,
which the compiler does not know. A register allocator that splits such a variable's live range inside the K loop and
restores it with a copy (at a loop's back edge, say), or spills it, makes the kernel read the register before the load has
landed - the results are then wrong now and then, and the late load hits whatever the register was reused for. Nothing in
the source can forbid that, so the generated code is checked, three ways:

1. Inside every basic block, exactly: a forward simulation of the load queue. State = the registers written by hand-issued
   loads of the block that no wait has covered yet, each with the number of vector-memory operations issued since (loads
   and stores retire in issue order and share one counter on this architecture); `s_waitcnt vmcnt(N)` retires every entry
   with at least N younger operations. Any other instruction that names a register still in the state - a copy of any
   width, an accumulator write, a scratch or buffer store, arithmetic, an overwrite - is reported, whatever its opcode.
2. Across the blocks of a K loop, by rule (the compiler's flag-driven control flow makes path-exact tracking across blocks
   report paths that cannot run): a block that neither drains the queue (`s_waitcnt vmcnt(0)`) nor has reached a
   hand-placed wait must not copy (`v_mov_b32`, `v_mov_b64`, `v_accvgpr_write_b32`) or store (`scratch_store`,
   `buffer_store`) a register that a 16-byte hand-issued load of the same loop writes. The one-word loads are the
   per-set scales, which the kernels copy on purpose once they have landed: they are exempt by register, not by opcode.
   A back-edge block that restores a split live range is exactly such a block.
3. The kernels' descriptors must show no scratch memory and no spilled vector registers.

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
VMEM = ("global_load", "global_store", "global_atomic", "buffer_load", "buffer_store", "buffer_atomic", "flat_load", "flat_store",
        "flat_atomic", "scratch_load", "scratch_store")
AGE_CAP = 64  # vmcnt is a 6-bit counter: older than 63 younger operations cannot be told apart


def _regs(tok):
    """Vector registers a token names: v7, v[4:7]; accumulator registers (a3, a[0:3]) are another file."""
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


def _blocks(body):
    """Basic blocks of one kernel: list of (label, instructions, successors). An instruction is (opcode, operand tokens,
    hand_issued, text)."""
    blocks, cur, inasm = [], {"label": "entry", "ins": [], "succ": [], "fall": True}, False
    for l in body[1:]:
        s = l.strip()
        if s.startswith(".Lfunc_end") or s.startswith(".section") or s.startswith(".rodata") or s.startswith(".p2align 6"):
            break
        m = re.match(r"^(\.LBB\d+_\d+):", l)
        if m:
            blocks.append(cur)
            cur = {"label": m.group(1), "ins": [], "succ": [], "fall": True}
            continue
        if "ASMSTART" in s:
            inasm = True
            continue
        if "ASMEND" in s:
            inasm = False
            continue
        if not s or s.startswith(";") or s.startswith("."):
            continue
        code = s.split(";")[0].strip()
        if not code:
            continue
        t = code.replace(",", " ").split()
        op = t[0]
        if op.startswith("s_cbranch"):
            cur["succ"].append(t[1])
            blocks.append(cur)  # the rest of the source block is a block of its own
            cur = {"label": cur["label"] + "+", "ins": [], "succ": [], "fall": True}
            continue
        if op == "s_branch":
            cur["succ"].append(t[1])
            cur["fall"] = False
            blocks.append(cur)
            cur = {"label": cur["label"] + "+", "ins": [], "succ": [], "fall": True, "dead": True}
            continue
        if op == "s_endpgm":
            cur["fall"] = False
            blocks.append(cur)
            cur = {"label": cur["label"] + "+", "ins": [], "succ": [], "fall": True, "dead": True}
            continue
        cur["ins"].append((op, t[1:], inasm, s))
    blocks.append(cur)
    return blocks


def _transfer(state, ins, report=None, where=""):
    """Runs one block over `state` (register -> younger vector-memory operations, smallest over all paths)."""
    state = dict(state)
    for op, toks, hand, text in ins:
        if op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", text)
            if m:
                n = int(m.group(1))
                state = {r: a for r, a in state.items() if a < n}
            continue
        named = set()
        for tok in toks:
            named |= _regs(tok)
        is_vmem = op.startswith(VMEM)
        is_hand_load = hand and op.startswith("global_load")
        dest = _regs(toks[0]) if (is_hand_load and toks) else set()
        touched = (named - dest) & set(state)  # a hand-issued load may target a register that still waits: loads land in order
        if touched and report is not None:
            report.append("%s: %s  [in flight: %s]" % (where, text, ", ".join("v%d" % r for r in sorted(touched))))
        if is_vmem:
            state = {r: min(a + 1, AGE_CAP) for r, a in state.items()}
        for r in dest:
            state[r] = 0
    return state


def _inflight_in_block(body):
    """Check 1. None when the kernel issues no loads by hand, else the instructions that touch a register in flight."""
    if not any("ASMSTART" in l for l in body):
        return None
    blocks = _blocks(body)
    if not any(hand and op.startswith("global_load") for b in blocks for op, _, hand, _ in b["ins"]):
        return None
    report = []
    for b in blocks:
        _transfer({}, b["ins"], report, b["label"])
    return report


def _loop_regions(body):
    """Labelled regions of a kernel with the loop (header label, depth) the compiler's comments put them in."""
    regions, cur, inasm = [], None, False
    for l in body[1:]:
        s = l.strip()
        m = re.match(r"^(\.LBB\d+_\d+):(.*)$", l) or re.match(r"^; %bb\.(\d+):(.*)$", l)
        if m:
            mm = re.search(r"Header=(BB\d+_\d+) Depth=(\d+)", m.group(2))
            cur = {"label": m.group(1), "loop": mm.group(1) if mm else None, "depth": int(mm.group(2)) if mm else 0, "ins": [], "fresh": True}
            regions.append(cur)
            continue
        if cur is None:
            continue
        if cur["fresh"] and s.startswith("; =>"):
            mm = re.search(r"Loop Header: Depth=(\d+)", s)
            if mm:
                cur["loop"], cur["depth"] = cur["label"].lstrip(".L"), int(mm.group(1))
            continue
        if "ASMSTART" in s:
            inasm = True
            continue
        if "ASMEND" in s:
            inasm = False
            continue
        if not s or s.startswith(";") or s.startswith("."):
            continue
        code = s.split(";")[0].strip()
        if not code:
            continue
        cur["fresh"] = False
        t = code.replace(",", " ").split()
        cur["ins"].append((t[0], t[1:], inasm, s))
    return regions


COPIES = ("v_mov_b32_e32", "v_mov_b64_e32", "v_accvgpr_write_b32")
STORES = ("scratch_store", "buffer_store")


def _loop_copies(body):
    """Check 2: (block, instruction) pairs of K-loop blocks that move a wide load destination before any wait."""
    loops = {}
    for r in _loop_regions(body):
        if r["loop"] and r["depth"] >= 2:
            loops.setdefault(r["loop"], []).append(r)
    out = []
    for regions in loops.values():
        wide = set()
        for r in regions:
            for op, toks, hand, _ in r["ins"]:
                if hand and op.startswith("global_load") and op != "global_load_dword":
                    wide |= _regs(toks[0])
        if not wide:
            continue
        for r in regions:
            if any(op == "s_waitcnt" and "vmcnt(0)" in text for op, _, _, text in r["ins"]):
                continue
            for op, toks, hand, text in r["ins"]:
                if hand and op == "s_waitcnt":
                    break  # what follows a hand-placed wait in its block are the reads the wait was placed for
                if hand:
                    continue
                src = set()
                for tok in (toks[1:] if op in COPIES else toks):
                    src |= _regs(tok)
                if (op in COPIES or op.startswith(STORES)) and src & wide:
                    out.append((r["label"], text))
    return out


def _spills(body):
    """Scratch memory and spilled registers from the kernel's descriptor and metadata comments."""
    bad = []
    for l in body:
        m = re.match(r"\s*\.amdhsa_private_segment_fixed_size\s+(\d+)", l)
        if m and int(m.group(1)) != 0:
            bad.append("scratch bytes %s" % m.group(1))
        m = re.match(r"\s*;\s*(ScratchSize|VGPR spill count|SGPR spill count):\s*(\d+)", l, re.I)
        if m and int(m.group(2)) != 0 and "SGPR" not in m.group(1).upper():
            bad.append("%s %s" % (m.group(1), m.group(2)))
    return bad


def _metadata_spills(text):
    """kernel name -> spilled vector registers, from the code object's metadata."""
    out, name = {}, None
    for l in text.split("\n"):
        m = re.match(r"\s*\.name:\s+(\S+)", l)
        if m:
            name = m.group(1)
        m = re.match(r"\s*\.vgpr_spill_count:\s+(\d+)", l)
        if m and name:
            out[name] = int(m.group(1))
    return out


def _snippet(*ins):
    body = ["k:"]
    for i in ins:
        if i.startswith("global_load") or i.startswith("HAND "):
            body += ["\t;;#ASMSTART", "\t" + i.replace("HAND ", ""), "\t;;#ASMEND"]
        else:
            body.append(i if i.endswith(":") or i.startswith(".LBB") else "\t" + i)
    return body


def test_checks_flag_a_copy_a_spill_and_an_early_read_and_accept_a_counted_wait():
    """The checks on hand-written snippets: a spill, arithmetic before the wait, the back-edge copy that once broke a kernel;
    and the shapes the kernels rely on (a wait that leaves younger loads in flight, a reload into a waiting register)."""
    def run(*ins):
        return _inflight_in_block(_snippet(*ins))

    load_a, load_b = "global_load_dwordx4 v[4:7], v1, s[2:3]", "global_load_dwordx4 v[8:11], v1, s[2:3] offset:16"
    assert run(load_a, "v_mov_b64_e32 v[20:21], v[4:5]", "s_waitcnt vmcnt(0)", "s_endpgm")
    assert run(load_a, "v_mov_b32_e32 v20, v6", "s_waitcnt vmcnt(0)", "s_endpgm")
    assert run(load_a, "v_accvgpr_write_b32 a3, v7", "s_waitcnt vmcnt(0)", "s_endpgm")
    assert run(load_a, "scratch_store_dwordx4 off, v[4:7], s32 offset:16", "s_waitcnt vmcnt(0)", "s_endpgm")
    assert run(load_a, "v_add_f32_e32 v4, v30, v31", "s_waitcnt vmcnt(0)", "s_endpgm")  # overwritten while the load is due
    # two loads, vmcnt(1) covers the older one only
    assert not run(load_a, load_b, "s_waitcnt vmcnt(1)", "v_mov_b32_e32 v20, v4", "s_waitcnt vmcnt(0)", "v_mov_b32_e32 v21, v8", "s_endpgm")
    assert run(load_a, load_b, "s_waitcnt vmcnt(1)", "v_mov_b32_e32 v21, v8", "s_waitcnt vmcnt(0)", "s_endpgm")
    # a store issued after the load counts as a younger operation: vmcnt(1) then covers the load
    assert not run(load_a, "global_store_dword v1, v30, s[4:5]", "s_waitcnt vmcnt(1)", "v_mov_b32_e32 v20, v4", "s_endpgm")
    # requesting into a register that still waits is what the rotating buffers do: the loads land in issue order
    assert not run(load_a, load_a, "s_waitcnt vmcnt(0)", "v_mov_b32_e32 v20, v4", "s_endpgm")

    # the loop rule: the load sits in the K loop's body, the copy in its back-edge block
    def loop(*back_edge):
        return _loop_copies(_snippet(
            ".LBB0_1:                                ; =>This Loop Header: Depth=1",
            ".LBB0_2:                                ;   Parent Loop BB0_1 Depth=1",
            "; =>  This Inner Loop Header: Depth=2",
            "HAND s_waitcnt vmcnt(1)", "v_mfma_f32_16x16x32_bf16 a[0:3], v[4:7], v[12:15], a[0:3]", load_a,
            "global_load_dword v30, v1, s[6:7]", "s_cbranch_scc1 .LBB0_4",
            ".LBB0_3:                                ;   in Loop: Header=BB0_2 Depth=2",
            *back_edge, "s_branch .LBB0_2",
            ".LBB0_4:                                ;   in Loop: Header=BB0_1 Depth=1", "s_waitcnt vmcnt(0)", "s_endpgm"))
    assert loop("v_mov_b64_e32 v[20:21], v[4:5]")
    assert loop("v_mov_b32_e32 v20, v7")
    assert loop("v_accvgpr_write_b32 a9, v5")
    assert loop("scratch_store_dword off, v6, s32")
    assert not loop("v_mov_b32_e32 v20, v30")          # the scale word, a one-word load: exempt by register
    assert not loop("v_mov_b64_e32 v[20:21], v[40:41]")  # not a load destination
    assert not loop("s_waitcnt vmcnt(0)", "v_mov_b64_e32 v[20:21], v[4:5]")  # a drain block


def _compile(tmp_path, source):
    if shutil.which("hipcc") is None:
        # every tier with ROCm installed has the compiler: a missing hipcc there is a failure, not a reason to skip
        if os.path.exists("/opt/rocm") or os.environ.get("CI"):
            pytest.fail("hipcc not on PATH although ROCm is installed")
        pytest.skip("no ROCm toolchain on this machine")
    asm = tmp_path / (os.path.splitext(source)[0] + ".s")
    r = subprocess.run(["hipcc", *FLAGS, "-o", str(asm), os.path.join(CSRC, source)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return asm.read_text()


def test_no_instruction_touches_a_register_with_a_load_in_flight(tmp_path):
    text = _compile(tmp_path, "prefill.hip")
    checked, bad, moved, spilled = 0, [], [], []
    vgpr_spills = _metadata_spills(text)
    assert len(vgpr_spills) >= 20
    for name, body in _kernels(text):
        hz = _inflight_in_block(body)
        if hz is None:
            continue
        checked += 1
        bad += ["%s %s" % (name, h) for h in hz[:4]]
        moved += ["%s %s: %s" % (name, blk, ins) for blk, ins in _loop_copies(body)[:4]]
        spilled += ["%s: %s" % (name, s) for s in _spills(body)]
        if vgpr_spills.get(name, 0):
            spilled.append("%s: %d vector registers spilled" % (name, vgpr_spills[name]))
    assert checked >= 20, "kernels with hand-issued loads found: %d" % checked
    assert not bad, "registers touched while a hand-issued load is in flight:\n" + "\n".join(bad[:24])
    assert not moved, "load destinations copied or stored in a K-loop block before any wait:\n" + "\n".join(moved[:24])
    assert not spilled, "kernels with hand-counted waits must not spill:\n" + "\n".join(spilled[:24])
