"""Builds niti_amd/libniti_gfx950.so from niti_amd/csrc/*.hip with hipcc for gfx950.

Usage: ``python -m niti_amd.build`` (cross-compiles without a GPU present)."""
from __future__ import annotations

import concurrent.futures as cf
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
SO = os.path.join(HERE, "libniti_gfx950.so")

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return obj


def build(verbose: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError("no HIP sources under " + CSRC)
    with cf.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    tmp = SO + ".tmp"
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    # a shared library links with undefined symbols left in it: resolve them all now, in a child process, so that
    # a library that cannot be loaded is never installed
    chk = subprocess.run([sys.executable, "-c", "import ctypes, os, sys; ctypes.CDLL(sys.argv[1], mode=os.RTLD_NOW)", tmp],
                         capture_output=True, text=True)
    if chk.returncode != 0:
        os.unlink(tmp)
        raise RuntimeError("the linked library does not load:\n" + chk.stderr[-2000:])
    os.replace(tmp, SO)
    if verbose:
        print("built", SO, os.path.getsize(SO), "bytes")
    return SO


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)
