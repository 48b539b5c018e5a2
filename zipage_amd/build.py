"""Build libzipage_hip.so (gfx950) in-tree with hipcc.

Run as ``python -m zipage_amd.build``.  The library is one shared object with a plain C
ABI (``include/zipage_hip.h``); it does not link against torch.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libzipage_hip.so")

# packed fp32 VALU ops are disabled on purpose (some forms misbehave on this fleet)
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # keep a*b+c as two roundings: the stages restate torch ops that round after each op
    "-ffp-contract=off",
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in proc.stderr.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stdout}\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = True, jobs: int | None = None) -> str:
    """Compile every source to an object file (in parallel) and link the shared object."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    extra = os.environ.get("ZP_EXTRA_HIPCC_FLAGS", "").split()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    compile_flags = [f for f in FLAGS if f != "-shared"]
    srcs = sources()
    objs = [os.path.join(objdir, os.path.basename(s)[:-4] + ".o") for s in srcs]
    jobs = jobs or min(len(srcs), os.cpu_count() or 1, 16)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda so: _run([hipcc, *compile_flags, *extra, "-c", so[0], "-o", so[1]], verbose),
                      zip(srcs, objs)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB + ".tmp"], verbose)
    os.replace(LIB + ".tmp", LIB)
    return LIB


if __name__ == "__main__":
    print(build())
