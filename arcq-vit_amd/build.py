"""Build recipe for ``libarcq_hip.so``: ``python -m arcq_vit_amd.build``.

hipcc cross-compiles for gfx950 without a GPU present.  The library lands next
to this file so that it travels with the source tree.  Every source file is
compiled to its own object (in parallel) and the objects are linked; with
``incremental=True`` an object newer than its source and every header is kept.
"""
from __future__ import annotations

import glob
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG_DIR)
_OBJ_DIR = os.path.join(_PKG_DIR, "csrc", "_obj")

COMPILE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-fvisibility=hidden",
    # Every float op rounds once unless the source says fma: results must equal the CPU restatement bit for bit.
    "-ffp-contract=off",
    # Keep the compiler from forming packed-fp32 VALU ops.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
LINK_FLAGS = ["--offload-arch=gfx950", "-shared", "-fPIC", "-fvisibility=hidden"]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # The host pass warns that it does not know the packed-fp32 target feature; that is expected.
    log = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}): {' '.join(cmd)}\n{log}")
    if verbose and log.strip():
        print(log)


def build(verbose: bool = False, incremental: bool = False, jobs: int = 6) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    srcs = sorted(glob.glob(os.path.join(_PKG_DIR, "csrc", "*.hip")))
    headers = glob.glob(os.path.join(_PKG_DIR, "csrc", "*.h")) + glob.glob(os.path.join(_ROOT, "include", "*.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    os.makedirs(_OBJ_DIR, exist_ok=True)
    out = os.path.join(_PKG_DIR, "libarcq_hip.so")
    objs, todo = [], []
    for s in srcs:
        o = os.path.join(_OBJ_DIR, os.path.basename(s)[:-4] + ".o")
        objs.append(o)
        fresh = (incremental and os.path.exists(o) and os.path.getmtime(o) > os.path.getmtime(s)
                 and os.path.getmtime(o) > newest_header)
        if not fresh:
            todo.append([hipcc, *COMPILE_FLAGS, "-I", os.path.join(_ROOT, "include"), "-c", s, "-o", o])
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        list(pool.map(lambda c: _run(c, verbose), todo))
    _run([hipcc, *LINK_FLAGS, "-o", out + ".tmp", *objs], verbose)
    os.replace(out + ".tmp", out)
    return out


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv, incremental="-i" in sys.argv))
