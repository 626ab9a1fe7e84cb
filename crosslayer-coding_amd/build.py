"""Builds libclt_hip.so (gfx950) from csrc/*.hip with hipcc.

    python crosslayer-coding_amd/build.py

The library lands in ``crosslayer-coding_amd/lib/``.  It has no torch dependency:
the C ABI in ``include/clt_hip.h`` takes raw device pointers and a hipStream_t.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBNAME = "libclt_hip.so"
ARCH = "gfx950"

# Packed-fp32 VALU forms are disabled for every device compile of this library.
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-pass-failed",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the CLT kernels cannot be built")
    return exe


def _run(cmd, verbose):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{out}")
    if verbose and out.strip():
        print(out)


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def build(verbose: bool = False, jobs: int = 4) -> str:
    """Compile every HIP source and link the shared library; returns its path."""
    hipcc = _hipcc()
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    cmds = []
    for src in sources():
        obj = os.path.join(objdir, src[:-4] + ".o")
        objs.append(obj)
        cmds.append([hipcc, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        list(ex.map(lambda c: _run(c, verbose), cmds))
    out = os.path.join(LIBDIR, LIBNAME)
    tmp = out + ".tmp"
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs], verbose)
    os.replace(tmp, out)
    return out


def library_path() -> str:
    return os.path.join(LIBDIR, LIBNAME)


if __name__ == "__main__":
    path = build(verbose="-v" in sys.argv)
    print(path)
