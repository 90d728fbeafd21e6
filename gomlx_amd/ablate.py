"""Timing-only ablations of the fused dequantise-in-LDS GEMM (csrc/gemm.hip).

Each variant is the shipped source with one part of a K step taken out by exact text substitution (the
substitution fails loudly when the source has moved on), compiled and linked with the product's other
objects into ``gomlx_amd/libgomlx_hipq_ablate_<name>.so``.  The variants compute WRONG results on purpose:
they exist to show, by the time that disappears with a part, what that part costs inside the running
kernel.  ``bench.py --ablation <name> --config c3`` times one; nothing else loads them.

    python -m gomlx_amd.ablate build [name ...]     # default: all
    python -m gomlx_amd.ablate clean
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys

from . import build as B

_STORE_X = "            x.template store_part<MASKED>(kk, nxt, k1, K, tid);\n"
_PART_W = "            wq.part(kk, w);\n"
_LOAD_X = "            x.load_part(kk, xb, fo);\n"
_STORE_W = """            if (kk == 1 || kk == 3) {
                const int o = (kk >> 1) * 8;
                wd[kk >> 1] = make_uint4(Op::pack(w[o], w[o + 1]) & wmask, Op::pack(w[o + 2], w[o + 3]) & wmask,
                                         Op::pack(w[o + 4], w[o + 5]) & wmask, Op::pack(w[o + 6], w[o + 7]) & wmask);
            }
"""
_KEEP_W = """            if (kk == 1 || kk == 3) {
                const int o = (kk >> 1) * 8;
                const uint32_t keep = (Op::pack(w[o], w[o + 1]) ^ Op::pack(w[o + 2], w[o + 3]) ^ Op::pack(w[o + 4], w[o + 5]) ^ Op::pack(w[o + 6], w[o + 7])) & wmask;
                asm volatile("" ::"v"(keep));
            }
"""
_LOAD_W = """        wq.load(wtile + (int64_t)kc * (BK / 32 * 34), ftail ? woff_t : woff, (uint32_t)wrun,
                min((int64_t)kc * (BK / 16) + wrun, n16 - 1));
    };
    auto stage_first"""
_NO_LOAD_W = """    };
    auto stage_first"""
_CONVERT = """        w[4 * i + 0] = sbyte0(a) * df;
        w[4 * i + 1] = sbyte1(a) * df;
        w[4 * i + 2] = sbyte2(a) * df;
        w[4 * i + 3] = sbyte3(a) * df;
"""
_NO_CONVERT = """        w[4 * i + 0] = __builtin_bit_cast(float, a);
        w[4 * i + 1] = __builtin_bit_cast(float, a ^ (uint32_t)d);
        w[4 * i + 2] = w[4 * i + 0];
        w[4 * i + 3] = w[4 * i + 1];
"""

_BLOCK = _STORE_X + _PART_W + _LOAD_X  # the staging a K step interleaves with each group of MFMAs


def _block(store_x=True, part_w=True, load_x=True):
    return (_BLOCK, (_STORE_X if store_x else "") + (_PART_W if part_w else "") + (_LOAD_X if load_x else ""))


# name: (what is taken out of the K loop, [(old, new), ...])
VARIANTS = {
    "no_convert": ("the int8 -> float arithmetic of the Q8_0 weights (bytes are passed on as bit patterns)", [(_CONVERT, _NO_CONVERT)]),
    "no_x_staging": ("activation loads and LDS stores", [_block(store_x=False, load_x=False)]),
    "no_x_stores": ("activation LDS stores (loads kept)", [_block(store_x=False)]),
    "no_x_loads": ("activation global loads (stores kept)", [_block(load_x=False)]),
    "no_w_staging": ("weight loads, conversion and LDS stores", [_block(part_w=False), (_STORE_W, ""), (_LOAD_W, _NO_LOAD_W)]),
    "no_w_loads": ("weight global loads (conversion and stores kept)", [(_LOAD_W, _NO_LOAD_W)]),
    "no_w_stores": ("weight LDS stores (loads and conversion kept)", [(_STORE_W, _KEEP_W)]),
    "no_staging": ("all staging: the loop is LDS fragment reads, MFMAs and barriers",
                   [_block(False, False, False), (_STORE_W, ""), (_LOAD_W, _NO_LOAD_W)]),
}


def lib_path(name: str) -> str:
    return os.path.join(B.HERE, f"libgomlx_hipq_ablate_{name}.so")


def variant_source(name: str) -> str:
    text = open(os.path.join(B.CSRC, "gemm.hip")).read()
    for old, new in VARIANTS[name][1]:
        if text.count(old) != 1:
            raise RuntimeError(f"ablation {name}: expected exactly one occurrence in gemm.hip of:\n{old}")
        text = text.replace(old, new)
    return text


def build_variant(name: str) -> str:
    out_dir = os.path.join(B.OBJ, "ablate")
    os.makedirs(out_dir, exist_ok=True)
    src = os.path.join(out_dir, f"gemm_{name}.hip")
    with open(src, "w") as f:
        f.write(variant_source(name))
    obj = os.path.join(out_dir, f"gemm_{name}.o")
    flags = [f for f in B.HIPCC_FLAGS if not f.startswith("-Rpass")]
    r = subprocess.run([B.hipcc(), *flags, "-I", B.CSRC, "-c", src, "-o", obj], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for ablation {name}:\n{r.stderr}")
    others = []
    for s in B.SOURCES:
        if s == "gemm.hip":
            continue
        o = os.path.join(B.OBJ, os.path.splitext(s)[0] + ".o")
        if not os.path.exists(o):
            raise RuntimeError(f"{o} is missing: build the product library first (python -m gomlx_amd.build)")
        others.append(o)
    r = subprocess.run([B.hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib_path(name), obj, *others], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed for ablation {name}:\n{r.stderr}")
    return lib_path(name)


def main(argv):
    if argv[:1] == ["clean"]:
        for p in glob.glob(lib_path("*")):
            os.remove(p)
        return 0
    if argv[:1] != ["build"]:
        sys.stderr.write(__doc__)
        return 2
    for name in argv[1:] or list(VARIANTS):
        print("built", build_variant(name), "--", "without", VARIANTS[name][0])
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
