"""Builds ``libmygrad_hip.so`` (gfx950 only) next to this file.

    python -m mygrad_amd.build          # compile what is out of date
    python -m mygrad_amd.build --force  # recompile everything

hipcc cross-compiles without a GPU, so this runs anywhere ROCm is installed.
"""

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
OBJDIR = os.path.join(HERE, "build")
LIBRARY = os.path.join(HERE, "libmygrad_hip.so")
SOURCES = ("runtime.hip", "pool.hip", "conv.hip", "conv_thin.hip", "elementwise.hip", "batchnorm.hip", "tiling.hip", "batched.hip")

# -packed-fp32-ops is switched off: the compiler must not form packed fp32 VALU
# instructions from ordinary float code.  (The host pass prints a harmless
# "not a recognized feature" note for it.)
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def _newest_header():
    stamps = [os.path.getmtime(os.path.join(INCLUDE, "mygrad_hip.h")), os.path.getmtime(__file__)]
    stamps += [os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC) if f.endswith(".h")]
    return max(stamps)


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(line for line in proc.stdout.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    return out


def build(force=False, verbose=False):
    """Compile the HIP sources and link the shared library; returns its path."""
    hipcc = _hipcc()
    os.makedirs(OBJDIR, exist_ok=True)
    header_stamp = _newest_header()
    jobs, objects = [], []
    for name in SOURCES:
        src = os.path.join(CSRC, name)
        obj = os.path.join(OBJDIR, name.replace(".hip", ".o"))
        objects.append(obj)
        stale = (
            force
            or not os.path.exists(obj)
            or os.path.getmtime(obj) < max(os.path.getmtime(src), header_stamp)
        )
        if stale:
            jobs.append([hipcc, *FLAGS, "-c", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=max(1, min(4, len(jobs)))) as pool:
        for out in pool.map(_run, jobs):
            if verbose and out.strip():
                print(out)
    if jobs or force or not os.path.exists(LIBRARY):
        out = _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", LIBRARY])
        if verbose and out.strip():
            print(out)
    return LIBRARY


if __name__ == "__main__":
    path = build(force="--force" in sys.argv, verbose=True)
    print(path)
