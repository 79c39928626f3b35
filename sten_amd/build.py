"""Build recipe for libnmg_hip.so (hipcc, gfx950 only).  Run as ``python -m sten_amd.build``."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libnmg_hip.so")
SOURCES = ["nmg_runtime.hip", "nmg_sparsify.hip", "nmg_spmm.hip", "nmg_smfmac.hip", "nmg_dense.hip",
           "nmg_densefrag.hip", "nmg_w4.hip", "nmg_pack.hip", "nmg_sddmm.hip", "nmg_perfect.hip", "nmg_gstream.hip", "nmg_sstream.hip", "nmg_ostream.hip"]
# bench.py's measurement aid: a library of its own, outside the product ABI
PROBE_LIB = os.path.join(HERE, "libnmg_probe.so")
PROBE_SOURCES = ["nmg_probe.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def build(verbose=False, jobs=8, check=True):
    """Compile every HIP source for gfx950 and link the shared library in-tree.  With ``check`` the
    compiled kernels that track their loads by hand are re-read (``isa_check``): a register touched
    while its load is in flight fails the build."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "_obj")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    for src in SOURCES + PROBE_SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        if src in SOURCES:
            objs.append(obj)
        cmd = [hipcc] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), file=sys.stderr)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB]
    subprocess.run(cmd, check=True)
    probe_objs = [os.path.join(objdir, src.replace(".hip", ".o")) for src in PROBE_SOURCES]
    subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + probe_objs + ["-o", PROBE_LIB], check=True)
    if check:
        from . import isa_check
        if isa_check.main([]) != 0:
            raise RuntimeError("isa_check: a kernel touches a register whose load is still in flight (see above)")
    return LIB


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        text = out.decode(errors="replace")
        # the host pass does not know the packed-fp32 target feature; that note is harmless
        text = "\n".join(l for l in text.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{text}")
        if text.strip():
            print(text, file=sys.stderr)


if __name__ == "__main__":
    print(build(verbose=True))
