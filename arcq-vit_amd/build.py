"""Build recipe for ``libarcq_hip.so``: ``python -m arcq_vit_amd.build``.

hipcc cross-compiles for gfx950 without a GPU present.  The library lands next
to this file so that it travels with the source tree.
"""
from __future__ import annotations

import glob
import os
import shutil
import subprocess
import sys

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG_DIR)

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-shared", "-fvisibility=hidden",
    # Every float op rounds once unless the source says fma: results must equal the CPU restatement bit for bit.
    "-ffp-contract=off",
    # Keep the compiler from forming packed-fp32 VALU ops.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose: bool = False) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    srcs = sorted(glob.glob(os.path.join(_PKG_DIR, "csrc", "*.hip")))
    out = os.path.join(_PKG_DIR, "libarcq_hip.so")
    cmd = [hipcc, *HIPCC_FLAGS, "-I", os.path.join(_ROOT, "include"), "-o", out + ".tmp", *srcs]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # The host pass warns that it does not know the packed-fp32 target feature; that is expected.
    log = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{log}")
    if verbose and log.strip():
        print(log)
    os.replace(out + ".tmp", out)
    return out


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
