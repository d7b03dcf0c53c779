"""Builds the HIP libraries for gfx950 with hipcc (no torch dependency).

Usage: ``python -m sga_amd.build`` -- compiles every product source of
``csrc/`` into ``sga_amd/libsga_hip.so`` (the C ABI of include/sga_hip.h and
nothing else) and ``csrc/bench_hooks.hip`` into ``sga_amd/libsga_hip_bench.so``
(timing observer + calibration kernels, loaded by bench.py only), both
in-tree.  -ffp-contract=off keeps every fp32 operation separately rounded (the
kernels place FMAs explicitly where the arithmetic recipe has one).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libsga_hip.so")
BENCH_LIB = os.path.join(HERE, "libsga_hip_bench.so")
SOURCES = ["fused_step.hip", "replay_group.hip", "select.hip", "elementwise.hip", "adamw.hip",
           "replay.hip", "runtime.hip", "scan.hip"]
BENCH_SOURCES = ["bench_hooks.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-ffp-contract=off", "-fno-fast-math",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    raise RuntimeError("hipcc not found")


def _stale(src, obj):
    """True unless ``obj`` is newer than ``src`` and every header of csrc/ and include/."""
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [src] + [os.path.join(d, f) for d in (CSRC, os.path.join(HERE, "..", "include"))
                    for f in os.listdir(d) if f.endswith((".hpp", ".h"))]
    return any(os.path.getmtime(d) > t for d in deps)


def build(verbose=True, jobs=8, extra=(), incremental=False):
    """Compile and link both libraries.  ``incremental`` (a convenience while
    editing) skips sources whose object file is newer than the source and all
    headers; the default compiles everything."""
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)

    def one(src):
        path = os.path.join(CSRC, src)
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        if incremental and not extra and not _stale(path, obj):
            return obj
        cmd = [hipcc, *FLAGS, *extra, "-c", path, "-o", obj]
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
        objs = list(ex.map(one, SOURCES + BENCH_SOURCES))
    for lib, group in ((LIB, objs[:len(SOURCES)]), (BENCH_LIB, objs[len(SOURCES):])):
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *group, "-o", lib]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
        if verbose:
            print(f"built {lib} from {len(group)} sources")
    return LIB


if __name__ == "__main__":
    build(extra=tuple(a for a in sys.argv[1:] if a.startswith("-D")),
          incremental="--incremental" in sys.argv[1:])
