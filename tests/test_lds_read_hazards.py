"""The operand reads of the direct-to-LDS convolution kernels are `asm volatile` ds_read_b128 instructions whose
guarding `s_waitcnt lgkmcnt(N)` stands in a LATER asm statement (so that the reads of the next fragments are in flight
while the matrix pipeline works on the previous ones).  The compiler knows nothing of that protocol: an instruction it
places between a read and its wait that touches the read's destination registers -- a copy at a loop edge, a spill, a
live-range split -- would see stale data, with no error.  This test makes that impossible to miss: it compiles the
kernels to device assembly with the flags of the build (`make isa`, 20 s) and walks every function:

* LDS reads complete in issue order, so after `s_waitcnt lgkmcnt(N)` all but the last N LDS operations have landed;
* between a hand-placed ds_read_b128 and the wait that covers it, NO other kind of instruction may read or write any
  of its four destination registers, and no later read may take its ADDRESS from them.  (A later hand-placed read
  into the SAME destination is allowed: LDS data returns in issue order, so the register ends up with the later
  read's data; the compiler shares a register between reads only when the earlier value is never used -- the
  prefetch of a tile that does not exist behind the last step.)
* at a loop edge -- a backward branch, the label it jumps to, the end of the function -- nothing hand-placed may be
  in flight: that is where the compiler places copies.  A forward branch (an `if` around the prefetch of the next
  tile) is walked straight through, reads of the skipped block included: the waits behind it are then checked
  against the path with MORE reads in flight, and a wait that is sufficient for that path is sufficient for the
  other.

Scalar memory loads share the counter and return out of order, so a function that issues one while hand-placed reads
are in flight is reported as well (none does).
"""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "sirius_amd", "csrc")

REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")


def vregs(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(3) is not None:
            out.add(int(m.group(3)))
        else:
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    return out


def check_function(name, lines):
    """Returns (hand-placed reads seen, list of problems)."""
    problems, seen = [], 0
    label_at = {}
    for no, raw in lines:
        m = re.match(r"^(\.L\w+):", raw.strip())
        if m:
            label_at[m.group(1)] = no
    loop_heads = set()
    for no, raw in lines:
        line = raw.split("//")[0].strip()
        if line.startswith(("s_cbranch", "s_branch")):
            target = line.split()[-1]
            if target in label_at and label_at[target] <= no:
                loop_heads.add(target)
    fifo = []            # LDS operations in flight, in issue order: (set of destination registers or None, line number)
    in_asm = False

    def hand_placed():
        return [f for f in fifo if f[0] is not None]

    for no, raw in lines:
        line = raw.split("//")[0].strip()
        if line.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if line.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not line or (line.startswith((";", ".")) and not line.endswith(":")):
            continue
        if line.endswith(":"):
            if line[:-1] in loop_heads and hand_placed():
                problems.append(f"{name}: line {no}: loop head {line} entered with {len(hand_placed())} hand-placed LDS reads in flight")
                fifo = []
            continue
        op = line.split()[0]
        if op in ("s_endpgm", "s_setpc_b64") or op.startswith(("s_cbranch", "s_branch")):
            backward = op.startswith(("s_cbranch", "s_branch")) and line.split()[-1] in loop_heads
            if (backward or not op.startswith(("s_cbranch", "s_branch"))) and hand_placed():
                problems.append(f"{name}: line {no}: `{line}` with {len(hand_placed())} hand-placed LDS reads in flight")
                fifo = []
            continue
        if op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", line)
            if m:
                keep = int(m.group(1))
                fifo = fifo[len(fifo) - keep:] if keep else []
            continue
        in_flight = set().union(*[f[0] for f in hand_placed()]) if hand_placed() else set()
        if op.startswith(("s_load", "s_buffer_load")) and in_flight:
            problems.append(f"{name}: line {no}: scalar load while hand-placed LDS reads are in flight")
        operands = line[len(op):]
        if op == "ds_read_b128" and in_asm:
            dst_txt, rest = operands.split(",", 1)
            dst, others = vregs(dst_txt), vregs(rest)
            if others & in_flight:
                problems.append(f"{name}: line {no}: `{line}` takes its address from an LDS read still in flight")
            fifo.append((dst, no))
            seen += 1
            continue
        touched = vregs(operands)
        if touched & in_flight:
            problems.append(f"{name}: line {no}: `{line}` touches v{sorted(touched & in_flight)} while the LDS read that fills "
                            f"them is in flight")
        if op.startswith("ds_"):
            fifo.append((None, no))     # the compiler's own LDS traffic: counted by the same counter, waited for by its own waits
    return seen, problems


def test_no_instruction_touches_an_lds_read_destination_before_its_wait():
    subprocess.run(["make", "-C", CSRC, "isa"], check=True, stdout=subprocess.DEVNULL)
    path = os.path.join(CSRC, "build", "conv_igemm.s")
    functions, current, name = {}, None, None
    with open(path) as f:
        for no, raw in enumerate(f, 1):
            m = re.match(r"^(_Z\w+):\s*(;.*)?$", raw)
            if m:
                name, current = m.group(1), []
                functions[name] = current
                continue
            if raw.startswith(".Lfunc_end"):
                current = None
                continue
            if current is not None:
                current.append((no, raw))
    total, problems, kernels = 0, [], 0
    for name, lines in functions.items():
        seen, bad = check_function(name, lines)
        total += seen
        kernels += 1 if seen else 0
        problems += bad
    assert kernels >= 20 and total >= 1000, (kernels, total)     # every direct-to-LDS tiling was seen
    assert not problems, "\n".join(problems[:20])
    print(f"{total} hand-placed LDS reads in {kernels} kernels: every one is untouched until its wait")


def test_the_checker_sees_a_planted_hazard():
    """The checker on four lines of assembly with the hazard in them, and on the same lines without."""
    bad = ["\t;;#ASMSTART", "\tds_read_b128 v[8:11], v2 offset:64", "\t;;#ASMEND", "\tv_mov_b32_e32 v20, v9",
           "\t;;#ASMSTART", "\ts_waitcnt lgkmcnt(0)", "\t;;#ASMEND", "\tv_mov_b32_e32 v21, v9", "\ts_endpgm"]
    seen, problems = check_function("planted", list(enumerate(bad, 1)))
    assert seen == 1 and len(problems) == 1 and "line 4" in problems[0]
    good = [l for i, l in enumerate(bad) if i != 3]
    assert check_function("clean", list(enumerate(good, 1))) == (1, [])
    # a counted wait: two reads in flight, lgkmcnt(1) releases the first only
    two = ["\t;;#ASMSTART", "\tds_read_b128 v[8:11], v2", "\t;;#ASMEND", "\t;;#ASMSTART", "\tds_read_b128 v[12:15], v3",
           "\t;;#ASMEND", "\ts_waitcnt lgkmcnt(1)", "\tv_add_f32_e32 v30, v8, v8", "\tv_add_f32_e32 v31, v12, v12",
           "\ts_waitcnt lgkmcnt(0)", "\ts_endpgm"]
    seen, problems = check_function("counted", list(enumerate(two, 1)))
    assert seen == 2 and len(problems) == 1 and "line 9" in problems[0]
    # a loop edge with a read in flight; the same read behind a forward branch is walked through
    edge = [".LBB0_1:", "\t;;#ASMSTART", "\tds_read_b128 v[8:11], v2", "\t;;#ASMEND", "\ts_cbranch_scc1 .LBB0_1", "\ts_endpgm"]
    assert "in flight" in check_function("edge", list(enumerate(edge, 1)))[1][0]
    fwd = ["\ts_cbranch_scc1 .LBB0_2", "\t;;#ASMSTART", "\tds_read_b128 v[8:11], v2", "\t;;#ASMEND", ".LBB0_2:",
           "\ts_waitcnt lgkmcnt(0)", "\tv_mov_b32_e32 v1, v8", "\ts_endpgm"]
    assert check_function("forward", list(enumerate(fwd, 1))) == (1, [])
    # an address taken from a register that is still being filled
    addr = ["\t;;#ASMSTART", "\tds_read_b128 v[8:11], v2", "\t;;#ASMEND", "\t;;#ASMSTART", "\tds_read_b128 v[12:15], v9",
            "\t;;#ASMEND", "\ts_waitcnt lgkmcnt(0)", "\ts_endpgm"]
    assert "address" in check_function("addr", list(enumerate(addr, 1)))[1][0]
