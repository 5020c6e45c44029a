"""Compiles the HIP sources under csrc/ into libhsa_gfx950.so (gfx950 only)."""
from __future__ import annotations

import concurrent.futures as cf
import glob
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libhsa_gfx950.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed fp32 VALU ops are switched off for every device compile
CFLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-Wno-unused-result",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _compile(src: str, extra) -> str:
    obj = os.path.join(CSRC, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC] + CFLAGS + list(extra) + ["-c", src, "-o", obj]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj


def build_library(extra_flags=(), jobs: int = 8, verbose: bool = False) -> str:
    """Always recompiles every source and relinks the shared library."""
    srcs = sources()
    with cf.ThreadPoolExecutor(max_workers=min(jobs, len(srcs))) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra_flags), srcs))
    cmd = [HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB_PATH] + objs
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("link failed:\n" + p.stdout)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build_library(verbose=True)
