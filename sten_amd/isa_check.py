"""Static check of the compiled kernels that track memory loads by hand.

Some kernels of this library issue their global loads as instruction statements and wait for them
with a counted ``s_waitcnt vmcnt(N)`` of their own.  The compiler does not know that the
destination registers of such a load are in flight: if it copies, spills or re-uses one of them
between the load and the wait that covers it, the kernel reads stale data now and then, with no
error.  This tool re-reads the device assembly the compiler produced and proves, per kernel, that

  * no instruction touches a register that a still-outstanding load will write (a spill of such a
    register is an instruction that reads it), and
  * no loop that streams operands holds scratch traffic, which would break the per-step count
    of operations the waits rely on (spills outside those loops are reported, not refused),

by simulating the in-order vector-memory counter along every kernel (loop bodies are walked twice,
so the state a loop carries into its next iteration is checked too).

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
}

REG = re.compile(r"\b([va])(\d+)\b|\b([va])\[(\d+):(\d+)\]")
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
    """[(kind, payload)] with kind in label / inst."""
    prog = []
    for raw in body:
        line = raw.split(";")[0].rstrip() if not raw.strip().startswith(";;#") else ""
        if not line.strip():
            continue
        m = LABEL.match(line.strip())
        if m and not line.startswith("\t"):
            prog.append(("label", m.group(1)))
            continue
        t = line.strip()
        if t.startswith("."):
            continue
        prog.append(("inst", t))
    return prog


notes = []


def check_kernel(name, body):
    """List of problems of one kernel (empty = clean); remarks that are no problems go to `notes`."""
    prog = parse(body)
    labels = {p[1]: i for i, p in enumerate(prog) if p[0] == "label"}
    problems = []
    seen = set()

    def step(inst, queue, where):
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
            if is_load and not to_lds:
                first = inst.split(None, 1)[1].split(",")[0]
                dest = regs_of(first)
            # the address / data registers it reads must not be in flight either
            for entry in queue:
                hit = entry & (touched - dest) if dest else entry & touched
                if hit:
                    problems.append(f"{where}: `{inst}` reads {sorted(hit)[:4]} while a load into them is outstanding")
            # a load into registers that an older outstanding load also writes would be ordered by the
            # hardware (in-order return), not a hazard
            queue.append(dest)
            return
        for entry in queue:
            hit = entry & touched
            if hit and (where, inst) not in seen:
                seen.add((where, inst))
                problems.append(f"{where}: `{inst}` touches {sorted(hit)[:4]} while a load into them is outstanding")

    # linear walk; at a backward branch, walk the loop body once more with the state at the branch
    queue = []
    i = 0
    revisited = set()
    while i < len(prog):
        kind, payload = prog[i]
        if kind == "inst":
            step(payload, queue, f"{name[:60]} @{i}")
            m = re.match(r"s_cbranch_\w+\s+(\S+)|s_branch\s+(\S+)", payload)
            if m:
                target = m.group(1) or m.group(2)
                if target in labels and labels[target] < i and (target, i) not in revisited:
                    revisited.add((target, i))
                    q2 = list(queue)
                    for j in range(labels[target], i):
                        if prog[j][0] == "inst":
                            step(prog[j][1], q2, f"{name[:60]} @{j} (second iteration)")
        i += 1
    # Spills: a spilled register with a load in flight is caught above (the scratch operation reads
    # it).  Scratch traffic inside a loop that streams operands would also disturb the counted
    # waits' budget of operations per step, so there it is an error; before and after the loops
    # (a value parked across the product) it is only reported.
    loops = []
    for i, (kind, payload) in enumerate(prog):
        if kind != "inst":
            continue
        m = re.match(r"s_cbranch_\w+\s+(\S+)|s_branch\s+(\S+)", payload)
        if m:
            target = m.group(1) or m.group(2)
            if target in labels and labels[target] < i:
                loops.append((labels[target], i))
    for i, (kind, payload) in enumerate(prog):
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
