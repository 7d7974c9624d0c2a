"""Build ``csrc/liboi_kernels.so`` for gfx950 with hipcc (``python -m open_instruct_amd.build``).

The shared object is built in-tree so that it travels with the source tree; nothing is compiled
at import time.
"""

from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
SOURCES = ["oi_rowwise.hip", "oi_loss.hip", "oi_pack.hip", "oi_lmhead.hip"]
OUTPUT = os.path.join(CSRC, "liboi_kernels.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # hipcc's auto-generated packed fp32 instructions are switched off for every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]  # fmt: skip


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def build(verbose: bool = False) -> str:
    """Compile every ``.hip`` source and link the shared library; returns its path."""
    objs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        noise = "is not a recognized feature for this target"
        err = "\n".join(line for line in res.stderr.splitlines() if noise not in line)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        objs.append(obj)
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", OUTPUT]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    for obj in objs:
        os.remove(obj)
    return OUTPUT


if __name__ == "__main__":
    print(build(verbose=True))
