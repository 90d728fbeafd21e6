"""Builds libgomlx_hipq.so (gfx950 only) in-tree with hipcc.

``python -m gomlx_amd.build`` compiles every translation unit under ``csrc/`` and links
them into ``gomlx_amd/libgomlx_hipq.so``.  Cross-compiles without a GPU.
"""
from __future__ import annotations

import json
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "build")
LIB = os.path.join(HERE, "libgomlx_hipq.so")
YARDSTICK_LIB = os.path.join(HERE, "libgq_yardstick.so")  # read-only kernels for the benchmark; not part of the product library

HOST = os.path.join(HERE, "host")
HOST_TEST = os.path.join(HOST, "build", "hipq_backend_test")
WORKSPACE_TEST = os.path.join(HOST, "build", "workspace_test")

# (the units that take longest to compile come first: they are the critical path of the parallel build)
SOURCES = ["gemm.hip", "gemm_dma.hip", "mlp.hip", "gemv_ks.hip", "api.hip", "dequant.hip", "gemv.hip", "gemv_xs.hip", "mmq.hip"]

# -packed-fp32-ops (note the minus): keep hipcc from forming v_pk_*_f32 instructions.
# -ffp-contract=off: dequantisation must round every fp32 operation on its own; fused
# multiply-adds are written explicitly (fmaf) where they are wanted.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
    "-Rpass-analysis=kernel-resource-usage",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _kernel_resources(stderr: str) -> dict:
    """Per-kernel register and scratch use from the compiler's resource-usage remarks."""
    out, name = {}, None
    for line in stderr.splitlines():
        m = re.search(r"remark: .*Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            out[name] = {}
            continue
        m = re.search(r"remark: .*?\s(VGPRs|AGPRs|ScratchSize \[bytes/lane\]|Occupancy \[waves/SIMD\]|LDS Size \[bytes/block\]): (\d+)", line)
        if m and name:
            out[name][m.group(1).split(" ")[0]] = int(m.group(2))
    return out


def _compile(src: str):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    noise = ("packed-fp32-ops", "target feature", "remark:")
    lines = r.stderr.splitlines()
    warn = "\n".join(l for i, l in enumerate(lines) if l.strip() and not any(n in l for n in noise)
                     and not (i > 0 and "remark:" in lines[i - 1]) and not (i > 1 and "remark:" in lines[i - 2]))
    if "warning" in warn:
        sys.stderr.write(warn + "\n")
    res = _kernel_resources(r.stderr)
    # A kernel that spills registers to scratch memory runs one to two orders of magnitude slower
    # than intended (it has happened when the compiler stopped inlining a kernel's lambdas): treat
    # it as a build error rather than ship it.
    spilled = {k: v["ScratchSize"] for k, v in res.items() if v.get("ScratchSize", 0) > 0}
    if spilled:
        raise RuntimeError(f"{src}: kernels use scratch memory (bytes per lane): {spilled}")
    return obj, res


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [o for o, _ in results]
    resources = {}
    for _, res in results:
        resources.update(res)
    with open(os.path.join(OBJ, "kernel_resources.json"), "w") as f:
        json.dump(resources, f, indent=1, sort_keys=True)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    cmd = [hipcc(), *[f for f in HIPCC_FLAGS if not f.startswith("-Rpass")], "-shared", os.path.join(CSRC, "yardstick.hip"), "-o", YARDSTICK_LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"yardstick build failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {YARDSTICK_LIB}")
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
    # the scratch-memory bookkeeping against fake device hooks (host only, no HIP)
    cmd = ["g++", "-O1", "-std=c++17", "-Wall", "-Wextra", "-pthread", os.path.join(HOST, "workspace_test.cpp"), "-o", WORKSPACE_TEST]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"workspace test build failed:\n{r.stdout}\n{r.stderr}")
    if r.stderr.strip():
        sys.stderr.write(r.stderr)
    if verbose:
        print(f"built {WORKSPACE_TEST}")
    build_sanitized(verbose)
    return HOST_TEST


SANITIZED = {
    # binary: (source, sanitizer flags, links the library)
    "workspace_test_tsan": ("workspace_test.cpp", ["-fsanitize=thread"], False),
    "workspace_test_asan": ("workspace_test.cpp", ["-fsanitize=address,undefined", "-fno-sanitize-recover=all"], False),
    "hipq_backend_test_asan": ("hipq_backend_test.cpp", ["-fsanitize=address,undefined", "-fno-sanitize-recover=all"], True),
}


def sanitized_path(name: str) -> str:
    return os.path.join(HOST, "build", name)


def build_sanitized(verbose: bool = True) -> dict:
    """The host-only test programs again under ThreadSanitizer (the two-threads-on-one-stream bookkeeping of the scratch
    pool) and under AddressSanitizer + UndefinedBehaviorSanitizer (pool bookkeeping; the host layer's graph-build rules).
    Host code only: the device library they link is the ordinary build."""
    os.makedirs(os.path.join(HOST, "build"), exist_ok=True)
    out = {}
    for name, (src, flags, links) in SANITIZED.items():
        cmd = ["g++", "-O1", "-g", "-fno-omit-frame-pointer", "-std=c++17", "-Wall", "-Wextra", "-pthread", *flags,
               os.path.join(HOST, src), "-o", sanitized_path(name)]
        if links:
            cmd += ["-L" + HERE, "-lgomlx_hipq", "-Wl,-rpath,$ORIGIN/../..", "-Wl,-rpath,/opt/rocm/lib"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"{name} build failed:\n{r.stdout}\n{r.stderr}")
        out[name] = sanitized_path(name)
        if verbose:
            print(f"built {out[name]}")
    return out


if __name__ == "__main__":
    build()
