"""Builds libdmoe_hip.so (gfx950) from disagmoe_amd/csrc with hipcc.

Usage: ``python -m disagmoe_amd.build`` (or ``__graft_entry__.build()``).  The
library is written next to this file so that it travels with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libdmoe_hip.so")
SOURCES = ["gmm_wave128_fp8.hip", "gmm_wave128.hip", "gmm_tile256.hip", "gmm_tile256_fp8.hip", "gmm_direct_bf16.hip", "gmm_direct_bf16_small.hip", "gmm_direct_fp8.hip", "gmm.hip", "route.hip", "topk.hip", "rows.hip",
           "meta.hip"]
ARCH = "gfx950"

FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", "-Wno-inline-asm",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP library cannot be built")
    return exe


def build(verbose: bool = True, jobs: int = 4, extra_flags=(), out: str = LIB_PATH, tag: str = "") -> str:
    """Compile and link.  ``extra_flags``/``out``/``tag`` build a second copy of the library next to the default
    one (its objects go to ``build<tag>/``)."""
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build" + tag)
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src: str) -> str:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
        if verbose and res.stderr.strip():
            # hipcc's host pass warns that it does not know packed-fp32-ops: harmless
            lines = [l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l]
            if lines:
                print("\n".join(lines), file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    tmp = out + ".tmp"
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    print(build())
