"""Builds libgomlx_hipq.so (gfx950 only) in-tree with hipcc.

``python -m gomlx_amd.build`` compiles every translation unit under ``csrc/`` and links
them into ``gomlx_amd/libgomlx_hipq.so``.  Cross-compiles without a GPU.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "build")
LIB = os.path.join(HERE, "libgomlx_hipq.so")

HOST = os.path.join(HERE, "host")
HOST_TEST = os.path.join(HOST, "build", "hipq_backend_test")

SOURCES = ["api.hip", "dequant.hip", "gemv.hip", "gemv_xs.hip", "gemv_ks.hip", "mmq.hip", "gemm.hip"]

# -packed-fp32-ops (note the minus): keep hipcc from forming v_pk_*_f32 instructions.
# -ffp-contract=off: dequantisation must round every fp32 operation on its own; fused
# multiply-adds are written explicitly (fmaf) where they are wanted.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    noise = ("packed-fp32-ops", "target feature")
    warn = "\n".join(l for l in r.stderr.splitlines() if l.strip() and not any(n in l for n in noise))
    if "warning" in warn:
        sys.stderr.write(warn + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    build_host_test(verbose)
    return LIB


def build_host_test(verbose: bool = True) -> str:
    """Compiles the C++ host layer's test program (host code only) against the library."""
    os.makedirs(os.path.dirname(HOST_TEST), exist_ok=True)
    cmd = ["g++", "-O1", "-std=c++17", "-Wall", "-Wextra", os.path.join(HOST, "hipq_backend_test.cpp"), "-o", HOST_TEST,
           "-L" + HERE, "-lgomlx_hipq", "-Wl,-rpath,$ORIGIN/../..", "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"host test build failed:\n{r.stdout}\n{r.stderr}")
    if r.stderr.strip():
        sys.stderr.write(r.stderr)
    if verbose:
        print(f"built {HOST_TEST}")
    return HOST_TEST


if __name__ == "__main__":
    build()
