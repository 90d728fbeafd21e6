"""Timing-only ablations of the fused dequantise-in-LDS GEMM (csrc/gemm.hip; names gemm_*, timed on --config c3 with
GOMLX_HIPQ_TWO_PASS_MIN_ROWS=100000 in the environment, which sends that shape through the fused kernel)
and of the Q4_K split-K route (csrc/mmq.hip; names q4k_*, timed on --config c2) and of the decode GEMV (csrc/gemv_ks_body.hpp; names ks_*, timed on
--config c0 / c1: single calls only, the batched and extended kernels live in other units).

Each variant is the shipped source with one part taken out by exact text substitution (the substitution
fails loudly when the source has moved on), compiled and linked with the product's other objects into
``gomlx_amd/libgomlx_hipq_ablate_<name>.so``.  The variants compute WRONG results on purpose: they exist
to show, by the time that disappears with a part, what that part costs inside the running kernel.
``bench.py --ablation <name> --config c3|c2`` times one; nothing else loads them.

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


_Q4K_IMAGE = """            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(img + i * 1024 + lane * 16),
                                             (__attribute__((address_space(3))) void *)(lds + i0 * 1024), 16, 0, 0);
"""
_Q4K_FETCH0 = "    if (par < nsb) fetch(par);\n"
_Q4K_FETCH = "        if (sbl + kParts < nsb) fetch(sbl + kParts);\n"
_Q4K_CONTRACT = "        q4k_contract_sb<false>(cur, lds, lds + xs_off + sbl * (kMT * 16), nullptr, sbl, kg, col, magic, acc);\n"
_Q4K_KEEP = '        asm volatile("" ::"v"(cur.hd.x), "v"(cur.c[0].x), "v"(cur.c[1].x), "v"(cur.c[2].x), "v"(cur.c[3].x), "v"(magic));\n'
_Q4K_PARTIAL = """            if (m < M) partial[((int64_t)slice * M + m) * set.ntot + set.n0[prob] + n] = v;
        }
    }
}

// ---- several tiles of 32 batch rows per weight tile"""
_Q4K_NO_PARTIAL = """            asm volatile("" ::"v"(v));
        }
    }
}

// ---- several tiles of 32 batch rows per weight tile"""
_Q4K_TILES_IMAGE = "    auto stage = [&](int sb, int h) __attribute__((always_inline)) {\n        uint8_t *dst = lds + h * L::kStageBytes;\n        for (int i = wave; i < NT * 8; i += G::kWaves) {\n"
_Q4K_TILES_NO_IMAGE = "    auto stage = [&](int sb, int h) __attribute__((always_inline)) {\n        uint8_t *dst = lds + h * L::kStageBytes;\n        for (int i = wave; i < (sb == 0 ? NT * 8 : 0); i += G::kWaves) {\n"
_Q4K_TILES_CONTRACT = "        q4k_tiles_half<NT, 0>(cur, lds, kg, col, magic, p1);\n"
_Q4K_XPREP = """    if (int rc = x_is_bf16 ? (fine ? prep(mmq_xprep_kernel<true, 1>) : prep(mmq_xprep_kernel<true, 2>))
                           : (fine ? prep(mmq_xprep_kernel<false, 1>) : prep(mmq_xprep_kernel<false, 2>)))
        return rc;
"""
_Q4K_REDUCE = "    if (count == 1) return launch_mmq_reduce(partial, partial2, xscale, nslices, M, K, N, items[0].bias, items[0].act, items[0].y, ex, s);\n"

_KS_STAGE = "                const Staged st = KS<T>::stage(p);\n"
_KS_NO_STAGE = """                Staged st;
                st.planes = make_uint4(__builtin_bit_cast(uint32_t, p.lo.x), __builtin_bit_cast(uint32_t, p.lo.y), __builtin_bit_cast(uint32_t, p.hi.x), __builtin_bit_cast(uint32_t, p.hi.y));
                st.scale = p.lo.z;
                st.sum = p.hi.z;
"""
_KS_DOT = "                for (int q = 0; q < R; q++) d[q] = KS<T>::dot(buf[jj], xq[q], xsc[q], xsm[q], c);\n"
_KS_NO_DOT = """                for (int q = 0; q < R; q++) {
                    const uint32_t *raw = reinterpret_cast<const uint32_t *>(&buf[jj]);
                    for (unsigned i = 0; i < sizeof(Raw) / 4; i++) asm volatile("" ::"v"(raw[i]));
                    d[q] = __builtin_bit_cast(float, xq[q][0].x ^ xq[q][7].w) + xsc[q][0] + xsm[q][0];
                }
"""
_KS_EPILOGUE = "    const int rows_out = dual ? rows_wg >> 1 : live * 8;\n"
_KS_NO_EPILOGUE = "    const int rows_out = (dual ? rows_wg >> 1 : live * 8) * (N < 0 ? 1 : 0);\n"
_KS_XFETCH = "            else KS<T>::x_fetch(reinterpret_cast<const float *>(xrow) + sl * kSliceValues, xl, r.a[i], r.b[i]);\n"
_KS_NO_XFETCH = "            else { r.a[i] = make_uint4(lane, sl, 3, 4); r.b[i] = make_uint4(5, 6, 7, xl); }\n"

# name: (source file, what is taken out, [(old, new), ...]) - or (unit, what, subs, edited header) when the text
# lives in a header that the unit includes
VARIANTS = {
    "gemm_no_convert": ("gemm.hip", "the int8 -> float arithmetic of the Q8_0 weights (bytes are passed on as bit patterns)", [(_CONVERT, _NO_CONVERT)]),
    "gemm_no_x_staging": ("gemm.hip", "activation loads and LDS stores", [_block(store_x=False, load_x=False)]),
    "gemm_no_x_stores": ("gemm.hip", "activation LDS stores (their loads are then dead code and go too)", [_block(store_x=False)]),
    "gemm_no_x_loads": ("gemm.hip", "activation global loads (stores kept)", [_block(load_x=False)]),
    "gemm_no_w_staging": ("gemm.hip", "weight loads, conversion and LDS stores", [_block(part_w=False), (_STORE_W, ""), (_LOAD_W, _NO_LOAD_W)]),
    "gemm_no_w_loads": ("gemm.hip", "weight global loads (conversion and stores kept)", [(_LOAD_W, _NO_LOAD_W)]),
    "gemm_no_w_stores": ("gemm.hip", "weight LDS stores (loads and conversion kept)", [(_STORE_W, _KEEP_W)]),
    "gemm_no_staging": ("gemm.hip", "all staging: the loop is LDS fragment reads, MFMAs and barriers",
                        [_block(False, False, False), (_STORE_W, ""), (_LOAD_W, _NO_LOAD_W)]),
    "ks_no_convert": ("gemv_ks.hip", "the conversion of the activations to fixed-point planes (loads and the LDS exchange kept)",
                      [(_KS_STAGE, _KS_NO_STAGE)], "gemv_ks_body.hpp"),
    "ks_no_x": ("gemv_ks.hip", "activation loads and their conversion (the LDS exchange of constants kept)",
                [(_KS_STAGE, _KS_NO_STAGE), (_KS_XFETCH, _KS_NO_XFETCH)], "gemv_ks_body.hpp"),
    "ks_no_dot": ("gemv_ks.hip", "the integer dot products (weight loads kept)", [(_KS_DOT, _KS_NO_DOT)], "gemv_ks_body.hpp"),
    "ks_no_epilogue": ("gemv_ks.hip", "the sum over the workgroup's wavefronts and the stores of y (the barrier stays)",
                       [(_KS_EPILOGUE, _KS_NO_EPILOGUE)], "gemv_ks_body.hpp"),
    "ks_no_store": ("gemv_ks.hip", "the global stores of y only (the sum over the wavefronts and the barrier stay)",
                    [("            y[at] = apply_act(act, t + (bias ? bias[row] : 0.f));\n",
                      '            asm volatile("" ::"v"(apply_act(act, t + (bias ? bias[row] : 0.f))), "v"(at));\n')], "gemv_ks_body.hpp"),
    "q4k_no_image": ("mmq.hip", "the copy of the slice's activation image into LDS (main kernel)", [(_Q4K_IMAGE, "            (void)img;\n")]),
    "q4k_no_weights": ("mmq.hip", "the weight loads of the main kernel (it contracts whatever LDS holds)", [(_Q4K_FETCH0, ""), (_Q4K_FETCH, "")]),
    "q4k_no_contract": ("mmq.hip", "unpacking and MFMAs of the main kernel (loads and LDS reads kept)", [(_Q4K_CONTRACT, _Q4K_KEEP)]),
    "q4k_main_empty": ("mmq.hip", "image copy, weight loads and contraction of the main kernel together (launch, barriers, LDS hand-over and partial stores remain)",
                       [(_Q4K_IMAGE, "            (void)img;\n"), (_Q4K_FETCH0, ""), (_Q4K_FETCH, ""), (_Q4K_CONTRACT, _Q4K_KEEP)]),
    "q4k_no_partials": ("mmq.hip", "the main kernel's stores of its partial sums", [(_Q4K_PARTIAL, _Q4K_NO_PARTIAL)]),
    "q4k_tiles_no_image": ("mmq.hip", "the image copies of the kernel for several batch tiles after its first super-block (barriers kept)",
                           [(_Q4K_TILES_IMAGE, _Q4K_TILES_NO_IMAGE)]),
    "q4k_tiles_no_contract": ("mmq.hip", "unpacking and MFMAs of the kernel for several batch tiles (loads, image copies and barriers kept)",
                              [(_Q4K_TILES_CONTRACT, _Q4K_KEEP),
                               ("        q4k_tiles_half<NT, 1>(cur, lds + L::kStageBytes, kg, col, magic, p1);\n", "")]),
    "q4k_no_xprep": ("mmq.hip", "the activation pre-pass launch", [(_Q4K_XPREP, "    (void)prep;\n")]),
    "q4k_no_reduce": ("mmq.hip", "the reduction launch", [(_Q4K_REDUCE, "    if (count == 1) return GQ_OK;\n")]),
}


def lib_path(name: str) -> str:
    return os.path.join(B.HERE, f"libgomlx_hipq_ablate_{name}.so")


def variant_source(name: str) -> str:
    """The edited text of the variant's file (the unit itself, or the header named as fourth entry)."""
    v = VARIANTS[name]
    src = v[3] if len(v) > 3 else v[0]
    text = open(os.path.join(B.CSRC, src)).read()
    for old, new in VARIANTS[name][2]:
        if text.count(old) != 1:
            raise RuntimeError(f"ablation {name}: expected exactly one occurrence in {src} of:\n{old}")
        text = text.replace(old, new)
    return text


def build_variant(name: str) -> str:
    out_dir = os.path.join(B.OBJ, "ablate")
    os.makedirs(out_dir, exist_ok=True)
    v = VARIANTS[name]
    src = os.path.join(out_dir, f"{name}.hip")
    if len(v) > 3:
        # the edited header goes into a directory of its own beside a copy of the unit: an #include "..." looks beside
        # the including file first
        out_dir = os.path.join(out_dir, name)
        os.makedirs(out_dir, exist_ok=True)
        src = os.path.join(out_dir, v[0])
        with open(os.path.join(out_dir, v[3]), "w") as f:
            f.write(variant_source(name))
        with open(src, "w") as f:
            f.write(open(os.path.join(B.CSRC, v[0])).read())
    else:
        with open(src, "w") as f:
            f.write(variant_source(name))
    obj = os.path.join(out_dir, f"{name}.o")
    flags = [f for f in B.HIPCC_FLAGS if not f.startswith("-Rpass")]
    r = subprocess.run([B.hipcc(), *flags, "-I", B.CSRC, "-c", src, "-o", obj], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for ablation {name}:\n{r.stderr}")
    others = []
    for s in B.SOURCES:
        if s == VARIANTS[name][0]:
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
        print("built", build_variant(name), "--", "without", VARIANTS[name][1])
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
