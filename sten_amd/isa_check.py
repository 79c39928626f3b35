"""Static check of the compiled kernels that track memory loads by hand.

Some kernels of this library issue their global loads as instruction statements and wait for them
with a counted ``s_waitcnt vmcnt(N)`` of their own.  The compiler does not know that the
destination registers of such a load are in flight: if it copies, spills or re-uses one of them
between the load and the wait that covers it, the kernel reads stale data now and then, with no
error.  This tool re-reads the device assembly the compiler produced and proves, per kernel, that

  * no instruction touches a register that a still-outstanding load will write (a spill of such a
    register is an instruction that reads it), and
  * no hand-issued load reads a scalar register less than five wait states after a vector
    instruction wrote it (the compiler keeps that distance for its own instructions only), and
  * no loop that streams operands holds scratch traffic, which would break the per-step count
    of operations the waits rely on, and no scratch load is issued while hand-issued loads are
    outstanding: the compiler's wait for it drains them all (other spills are reported, not
    refused),

by simulating the in-order vector-memory counter along every kernel (loop bodies are walked again
with the state their back edge carries, so what a loop hands to its next iteration is checked too).

    python -m sten_amd.isa_check                  # all sources that contain hand-issued loads
    python -m sten_amd.isa_check file.s --kernels dense_direct   # an assembly file made elsewhere

Exit status 0 = clean.  ``sten_amd.build`` runs it after compiling.
"""
import argparse
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
# sources whose kernels issue loads as instruction statements, and the kernels (substring of the
# mangled name) that do
CHECKED = {
    "nmg_densefrag.hip": ["dense16_direct_kernel"],
    "nmg_smfmac.hip": ["spmm_smfmac_direct_kernel", "decode_staged_kernel"],
    "nmg_w4.hip": ["w4_linear_staged_kernel"],
    "nmg_sddmm.hip": ["sddmm16_kernel"],
    "nmg_gstream.hip": ["gstream_kernel"],
    "nmg_sstream.hip": ["sstream_kernel"],
    "nmg_ostream.hip": ["ostream_kernel"],
}

REG = re.compile(r"\b([va])(\d+)\b|\b([va])\[(\d+):(\d+)\]")
SREG = re.compile(r"\bs(\d+)\b|\bs\[(\d+):(\d+)\]")
VMEM = re.compile(r"^(global|buffer|scratch|flat)_(load|store|atomic)")
LABEL = re.compile(r"^(\.?[A-Za-z_][\w.$]*):")


def regs_of(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(1):
            out.add((m.group(1), int(m.group(2))))
        else:
            for r in range(int(m.group(4)), int(m.group(5)) + 1):
                out.add((m.group(3), r))
    return out


def sregs_of(text):
    out = set()
    for m in SREG.finditer(text):
        if m.group(1):
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def scalar_hazards(name, prog):
    """A scalar register written by a vector instruction (a lane read that brings back a parked
    base, a compare) must rest five wait states before a vector-memory instruction reads it.  The
    compiler inserts them for its own instructions; it does not look into instruction statements,
    so the hand-issued loads are checked here, in layout order."""
    problems = []
    age = {}      # scalar register -> wait states since a vector instruction wrote it
    for i, (kind, inst, by_hand) in enumerate(prog):
        if kind != "inst":
            continue
        op = inst.split()[0]
        if by_hand and VMEM.match(op):
            young = sorted(r for r in sregs_of(inst) if age.get(r, 99) < 5)
            if young:
                problems.append(f"{name[:60]} @{i}: `{inst}` reads s{young[:4]} less than five wait states after a "
                                "vector instruction wrote them")
        states = 1
        if op == "s_nop":
            states = int(inst.split()[1], 0) + 1
        for r in list(age):
            age[r] += states
        if op.startswith("v_") and len(inst.split(None, 1)) > 1:
            first = inst.split(None, 1)[1].split(",")[0]
            for r in sregs_of(first):
                age[r] = 0
    return problems


def kernels_of(asm_text):
    """{mangled name: [instruction lines]} for every kernel of an assembly file."""
    out = {}
    lines = asm_text.split("\n")
    i = 0
    while i < len(lines):
        m = re.match(r"^(_Z\w+):", lines[i])
        if m:
            name = m.group(1)
            body = []
            i += 1
            while i < len(lines) and not lines[i].startswith("\t.end_amdhsa_kernel") \
                    and not lines[i].startswith(".Lfunc_end"):
                body.append(lines[i])
                i += 1
            out[name] = body
        i += 1
    return out


def parse(body):
    """[(kind, payload, by_hand)] with kind in label / inst; by_hand: the instruction stands inside
    an instruction statement of the source (between the compiler's ASMSTART / ASMEND marks)."""
    prog = []
    by_hand = False
    for raw in body:
        mark = raw.strip()
        if mark.startswith(";;#ASMSTART"):
            by_hand = True
        elif mark.startswith(";;#ASMEND"):
            by_hand = False
        line = raw.split(";")[0].rstrip() if not mark.startswith(";;#") else ""
        if not line.strip():
            continue
        m = LABEL.match(line.strip())
        if m and not line.startswith("\t"):
            prog.append(("label", m.group(1), False))
            continue
        t = line.strip()
        if t.startswith("."):
            continue
        prog.append(("inst", t, by_hand))
    return prog


notes = []


def check_kernel(name, body):
    """List of problems of one kernel (empty = clean); remarks that are no problems go to `notes`."""
    prog = parse(body)
    labels = {p[1]: i for i, p in enumerate(prog) if p[0] == "label"}
    problems = scalar_hazards(name, prog)
    seen = set()
    # Only the loads of instruction statements are tracked by register: the compiler waits for its
    # own loads itself, they only take their place in the queue.  (An assembly text without the
    # compiler's marks -- a test, a hand-written file -- has every load tracked.)
    marked = any(p[2] for p in prog)

    def step(inst, queue, where, by_hand=True):
        op = inst.split()[0]
        if op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", inst)
            if m:
                keep = int(m.group(1))
                if len(queue) > keep:
                    del queue[:len(queue) - keep]
            return
        touched = regs_of(inst)
        if VMEM.match(op):
            is_load = "_load" in op or "atomic" in op
            to_lds = "_lds_" in op or op.endswith("_lds")
            dest = set()
            if is_load and not to_lds and (by_hand or not marked):
                first = inst.split(None, 1)[1].split(",")[0]
                dest = regs_of(first)
            # A spill among hand-issued loads in flight: the compiler counts only its own operations, so
            # its wait for this one is a wait for everything requested before it -- the sets that
            # were meant to stay in flight are drained (correct, and several times slower).
            # (a spill *store* only adds one operation to the count: the waits behind it get more
            # conservative, and it is reported with the other spills)
            if op.startswith("scratch_load") and marked and any(queue):
                problems.append(f"{where}: `{inst}` is scratch traffic while hand-issued loads are outstanding")
            # the address / data registers it reads must not be in flight either
            for entry in queue:
                hit = entry & (touched - dest) if dest else entry & touched
                if hit:
                    problems.append(f"{where}: `{inst}` reads {sorted(hit)[:4]} while a load into them is outstanding")
            # a load into registers that an older outstanding load also writes would be ordered by the
            # hardware (in-order return), not a hazard
            queue.append(dest)
            if len(queue) > 63:          # the counter holds 63: older operations have completed
                del queue[:len(queue) - 63]
            return
        for entry in queue:
            hit = entry & touched
            if hit and (where, inst) not in seen:
                seen.add((where, inst))
                problems.append(f"{where}: `{inst}` touches {sorted(hit)[:4]} while a load into them is outstanding")

    # Walk in layout order, which for these kernels is execution order, with two corrections.  An
    # unconditional forward branch is followed (what lies behind it is never fallen into: a rotated
    # loop has its body there, entered from its header further down).  At a backward branch the
    # stretch from its target to the branch is walked twice more, each time with the state the
    # previous walk ended in: what a loop hands to its next iteration is checked too.  Conditional
    # forward branches (loop exits, guards) are not followed: their conditions are correlated in
    # ways a path search cannot see, and it would report paths that never run.
    flagged = set()

    def step_once(pc, inst, queue, looped):
        before = len(problems)
        step(inst, queue, f"{name[:60]} @{pc}" + (" (second iteration)" if looped else ""), prog[pc][2])
        if len(problems) > before:
            if pc in flagged:
                del problems[before:]
            else:
                flagged.add(pc)
                del problems[before + 1:]

    BR = re.compile(r"s_cbranch_\w+\s+(\S+)|s_branch\s+(\S+)")

    def walk(pc, stop, queue, looped, rewalks):
        """Walk from pc until `stop` (exclusive) is reached or passed; returns the queue at the end."""
        while pc < stop:
            kind, payload = prog[pc][0], prog[pc][1]
            if kind == "inst":
                step_once(pc, payload, queue, looped)
                m = BR.match(payload)
                if m:
                    target = m.group(1) or m.group(2)
                    if target in labels:
                        t = labels[target]
                        if t < pc and rewalks > 0 and (t, pc) not in done_loops:
                            done_loops.add((t, pc))
                            q2 = list(queue)
                            for _ in range(rewalks):
                                q2 = walk(t, pc + 1, q2, True, 0)
                        elif t > pc and m.group(2):
                            pc = t
                            continue
            pc += 1
        return queue

    done_loops = set()
    walk(0, len(prog), [], False, 2)
    # Spills: a spilled register with a load in flight is caught above (the scratch operation reads
    # it).  Scratch traffic inside a loop that streams operands would also disturb the counted
    # waits' budget of operations per step, so there it is an error; before and after the loops
    # (a value parked across the product) it is only reported.
    loops = []
    for i, (kind, payload, _) in enumerate(prog):
        if kind != "inst":
            continue
        m = re.match(r"s_cbranch_\w+\s+(\S+)|s_branch\s+(\S+)", payload)
        if m:
            target = m.group(1) or m.group(2)
            if target in labels and labels[target] < i:
                loops.append((labels[target], i))
    for i, (kind, payload, _) in enumerate(prog):
        if kind == "inst" and payload.startswith("scratch_"):
            inside = [lp for lp in loops if lp[0] <= i <= lp[1]
                      and any(prog[j][0] == "inst" and prog[j][1].startswith("global_load") for j in range(lp[0], lp[1]))]
            if inside:
                problems.append(f"{name[:60]} @{i}: `{payload}` spills inside a loop that streams operands")
            else:
                notes.append(f"{name[:60]} @{i}: `{payload}` (spill outside the streaming loops)")
    return problems


def assembly_of(source):
    """Device assembly of one HIP source, compiled with the flags of the library."""
    from .build import FLAGS
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        cmd = [hipcc] + FLAGS + ["--cuda-device-only", "-S", os.path.join(CSRC, source), "-o", out]
        subprocess.run(cmd, check=True, stdout=subprocess.PIPE, stderr=subprocess.PIPE)
        return open(out).read()


def check_text(asm_text, wanted):
    problems, checked = [], 0
    for name, body in kernels_of(asm_text).items():
        if not any(w in name for w in wanted):
            continue
        checked += 1
        problems += check_kernel(name, body)
    return checked, problems


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("asm", nargs="?", help="an assembly file (default: compile the checked sources)")
    ap.add_argument("--kernels", nargs="*", default=None, help="substrings of the kernel names to check")
    args = ap.parse_args(argv)
    total, problems = 0, []
    if args.asm:
        n, p = check_text(open(args.asm).read(), args.kernels or [""])
        total, problems = n, p
    else:
        for source, wanted in CHECKED.items():
            n, p = check_text(assembly_of(source), args.kernels or wanted)
            total += n
            problems += p
    for p in problems:
        print(p)
    for q in sorted(set(n.split(" @")[0] for n in notes)):
        print(f"note: {q}: spills outside the streaming loops")
    print(f"isa_check: {total} kernels, {len(problems)} problems")
    return 1 if problems else 0


if __name__ == "__main__":
    sys.exit(main())
