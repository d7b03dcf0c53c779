"""Builds libsga_hip.so for gfx950 with hipcc (no torch dependency).

Usage: ``python -m sga_amd.build`` -- compiles every ``csrc/*.hip`` into
``sga_amd/libsga_hip.so`` in-tree.  -ffp-contract=off keeps every fp32
operation separately rounded (the kernels place FMAs explicitly where the
arithmetic recipe has one).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libsga_hip.so")
SOURCES = ["runtime.hip", "scan.hip", "elementwise.hip", "adamw.hip",
           "select.hip", "fused_step.hip", "replay.hip", "replay_group.hip",
           "bench_hooks.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-ffp-contract=off", "-fno-fast-math",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    raise RuntimeError("hipcc not found")


def build(verbose=True, jobs=8, extra=()):
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]

    def one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
        if verbose and r.stderr.strip():
            # the host pass warns that it does not know packed-fp32-ops
            lines = [l for l in r.stderr.splitlines()
                     if "packed-fp32-ops" not in l and l.strip()]
            if lines:
                print("\n".join(lines), file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(one, srcs))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    return LIB


if __name__ == "__main__":
    build(extra=tuple(a for a in sys.argv[1:] if a.startswith("-D")))
