"""Builds libohara_decode.so (the HIP kernels + C ABI) for gfx950 with hipcc.

The library is built in-tree (``ohara_amd/lib/``); nothing is JIT-compiled at
import time.  ``python -m ohara_amd.build`` rebuilds it; ``--incremental`` recompiles
only the sources that are newer than their objects (or older than a header).
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")
LIB_PATH = os.path.join(LIB_DIR, "libohara_decode.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
_NOISE = "is not a recognized feature for this target"


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers_mtime() -> float:
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs += [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE) if f.endswith(".h")]
    return max(os.path.getmtime(h) for h in hs)


def _run(cmd: list[str]) -> str:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in proc.stderr.splitlines() if _NOISE not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{' '.join(cmd)}\n{err}")
    return err


def build_library(verbose: bool = False, incremental: bool = False, jobs: int = 8) -> str:
    """One object per source (compiled in parallel), then one link."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    hdr = _headers_mtime()
    todo, objs = [], []
    for src in sources():
        obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        fresh = (incremental and os.path.exists(obj) and os.path.getmtime(obj) >= os.path.getmtime(src)
                 and os.path.getmtime(obj) >= hdr)
        if not fresh:
            todo.append((src, obj))
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        errs = list(pool.map(lambda so: _run([HIPCC, *FLAGS, "-c", so[0], "-o", so[1]]), todo))
    errs.append(_run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]))
    if verbose:
        for e in errs:
            if e.strip():
                print(e, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True, incremental="--incremental" in sys.argv))
