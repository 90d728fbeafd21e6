"""CPU oracle for GoMLX's quantized Dense path -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the GPU product path never does.

Two independent restatements of the reference algorithm live here:

* ``np_*``  -- vectorised numpy (byte / integer arithmetic with array ops);
* ``c_*``   -- thin ctypes bindings of ``libggml_oracle.so`` (scalar C loops,
  built from ``ggml_oracle.c`` by ``oracle/Makefile``).

They are written differently on purpose so that each checks the other, and both are
pinned against the reference's own known-answer tests in ``tests/golden/``.

Pinning status: fp16 decode, Q8_0, Q4_0, IQ4_NL, dense, bias/activation and gather are
pinned (reference KATs + closed forms + brute force, see tests/test_oracle.py).
**Q4_K is PARITY UNPINNED at the reference**: its only implementation is in the
un-vendored module github.com/gomlx/compute v0.1.2 (reached from
ml/nn/quantized_dense.go:56); it is restated from the public GGML block_q4_K layout.
**Q6_K is PARITY UNPINNED** for the same reason (the reference only names the type,
docs/CHANGELOG.md:251-252); it is restated from the public GGML block_q6_K layout.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

Q4_0, Q8_0, Q4_K, Q6_K, IQ4_NL = 2, 8, 12, 14, 20
ACT_NONE, ACT_GELU, ACT_RELU, ACT_SILU, ACT_HARDSWISH, ACT_TANH = range(6)

_GEOM = {Q4_0: (18, 32), Q8_0: (34, 32), Q4_K: (144, 256), Q6_K: (210, 256), IQ4_NL: (18, 32)}

# Public GGML IQ4_NL table (compute.IQ4NLLookupTable, ml/ggml/dequant.go:130).
IQ4NL_LUT = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113],
                     dtype=np.float32)


def bytes_per_block(t: int) -> int:
    return _GEOM[t][0]


def values_per_block(t: int) -> int:
    return _GEOM[t][1]


def row_bytes(t: int, K: int) -> int:
    bpb, vpb = _GEOM[t]
    if K <= 0 or K % vpb:
        return 0
    return K // vpb * bpb


# --------------------------------------------------------------------------- numpy

def _f16(b: np.ndarray) -> np.ndarray:
    """u8[..., 2] little-endian -> f32[...] (Bitcast + ConvertDType, ml/ggml/dequant.go:63-66)."""
    return np.ascontiguousarray(b).view("<f2")[..., 0].astype(np.float32)


def np_dequantize(t: int, W: np.ndarray, K: int | None = None) -> np.ndarray:
    """ggml.Dequantize (ml/ggml/dequant.go:39-54): W [N, rowBytes] u8 -> [N, K] f32."""
    W = np.ascontiguousarray(W, dtype=np.uint8)
    N, rb = W.shape
    bpb, vpb = _GEOM[t]
    if rb % bpb:
        raise ValueError("row bytes not a whole number of blocks")
    nb = rb // bpb
    if K is not None and K != nb * vpb:
        raise ValueError("K does not match the row bytes")
    w = W.reshape(N, nb, bpb)
    if t == Q8_0:  # ml/ggml/dequant.go:58-78
        d = _f16(w[:, :, 0:2])[:, :, None]
        q = w[:, :, 2:34].view(np.int8).astype(np.float32)
        return (q * d).reshape(N, nb * 32)
    if t in (Q4_0, IQ4_NL):  # extractNibbleBlock, ml/ggml/dequant.go:83-98
        d = _f16(w[:, :, 0:2])[:, :, None]
        nib = w[:, :, 2:18]
        comb = np.concatenate([nib & 0x0F, nib >> 4], axis=2)
        if t == Q4_0:  # ml/ggml/dequant.go:104-115
            v = comb.astype(np.float32) - np.float32(8.0)
        else:  # ml/ggml/dequant.go:121-136
            v = IQ4NL_LUT[comb]
        return (v * d).reshape(N, nb * 32)
    if t == Q4_K:  # public GGML block_q4_K (parity unpinned at the reference)
        d = _f16(w[:, :, 0:2])
        dmin = _f16(w[:, :, 2:4])
        s = w[:, :, 4:16].astype(np.int32)
        sc = np.empty((N, nb, 8), np.int32)
        mn = np.empty((N, nb, 8), np.int32)
        sc[:, :, :4] = s[:, :, 0:4] & 63
        mn[:, :, :4] = s[:, :, 4:8] & 63
        sc[:, :, 4:] = (s[:, :, 8:12] & 0x0F) | ((s[:, :, 0:4] >> 6) << 4)
        mn[:, :, 4:] = (s[:, :, 8:12] >> 4) | ((s[:, :, 4:8] >> 6) << 4)
        qs = w[:, :, 16:144].reshape(N, nb, 4, 32)
        codes = np.stack([qs & 0x0F, qs >> 4], axis=3)  # [N, nb, 4, 2, 32] -> sub-block 2g+h
        codes = codes.reshape(N, nb, 8, 32).astype(np.float32)
        dsc = (d[:, :, None] * sc.astype(np.float32))[:, :, :, None]
        dm = (dmin[:, :, None] * mn.astype(np.float32))[:, :, :, None]
        return (dsc * codes - dm).astype(np.float32).reshape(N, nb * 256)
    if t == Q6_K:  # public GGML block_q6_K (parity unpinned at the reference)
        ql = w[:, :, 0:128].reshape(N, nb, 2, 2, 32)     # [half][which 32 bytes][l]
        qh = w[:, :, 128:192].reshape(N, nb, 2, 1, 32)   # [half][.][l]
        sc = w[:, :, 192:208].view(np.int8).astype(np.float32).reshape(N, nb, 2, 4, 2)  # [half][quadrant][l / 16]
        d = _f16(w[:, :, 208:210])
        lo = np.stack([ql & 0x0F, ql >> 4], axis=3)       # [N, nb, half, nibble, which, l]
        lo = lo.reshape(N, nb, 2, 4, 32)                  # quadrant = 2 * nibble + which
        shifts = np.array([0, 2, 4, 6], np.uint8).reshape(1, 1, 1, 4, 1)
        hi = (qh >> shifts) & 3                           # [N, nb, half, quadrant, l]
        q = (lo | (hi << 4)).astype(np.int32) - 32
        scale = np.repeat(sc, 16, axis=4)                 # [N, nb, half, quadrant, 32]
        ds = d[:, :, None, None, None] * scale
        return (ds * q.astype(np.float32)).astype(np.float32).reshape(N, nb * 256)
    raise ValueError(f"unsupported ggml type {t}")


def np_activation(act: int, v: np.ndarray) -> np.ndarray:
    """activation.Apply for the types with a backend enum (activation.go:58-75,161,195,222-243,274-286)."""
    from math import sqrt

    x = v.astype(np.float64)
    if act == ACT_NONE:
        return v.astype(np.float32)
    if act == ACT_RELU:
        r = np.maximum(x, 0.0)
    elif act == ACT_SILU:
        r = x / (1.0 + np.exp(-x))
    elif act == ACT_HARDSWISH:
        r = x * np.clip(x / 6.0 + 0.5, 0.0, 1.0)
    elif act == ACT_TANH:
        r = np.tanh(x)
    elif act == ACT_GELU:
        from scipy.special import erf

        r = x * 0.5 * (1.0 + erf(x / sqrt(2.0)))
    else:
        raise ValueError(f"unknown activation {act}")
    return r.astype(np.float32)


def np_qdense(t: int, x: np.ndarray, W: np.ndarray, bias: np.ndarray | None = None,
              act: int = ACT_NONE) -> np.ndarray:
    """ggml.DenseDecomposed (ml/ggml/dense.go:23-62), fp64 accumulation, x [..., K]."""
    x = np.asarray(x, dtype=np.float32)
    K = x.shape[-1]
    Wd = np_dequantize(t, W, K)
    y = x.reshape(-1, K).astype(np.float64) @ Wd.astype(np.float64).T
    if bias is not None:
        y = y + np.asarray(bias, np.float32).astype(np.float64)[None, :]
    y = np_activation(act, y.astype(np.float32))
    return y.reshape(x.shape[:-1] + (Wd.shape[0],))


def np_rmsnorm(x: np.ndarray, gain: np.ndarray | None = None, eps: float = 1e-6, gain_offset: float = 0.0) -> np.ndarray:
    """norm.RMSNorm over the last axis (ml/layers/norm/rmsnorm.go:78-113), evaluated in float64 and
    rounded once: an independent form of the C routine, which rounds node by node."""
    x64 = np.asarray(x, np.float32).astype(np.float64)
    r = np.sqrt(np.mean(x64 * x64, axis=-1, keepdims=True) + float(np.float32(eps)))
    y = x64 / r
    if gain is not None:
        y = y * (np.asarray(gain, np.float32).astype(np.float64) + float(np.float32(gain_offset)))
    return y.astype(np.float32)


def np_gated_ffn(t: int, x: np.ndarray, Wgate: np.ndarray, Wup: np.ndarray, bias_gate=None, bias_up=None, act: int = ACT_SILU,
                 norm: tuple | None = None) -> np.ndarray:
    """ff = activation(dense(xn, Wgate)) * dense(xn, Wup) (ml/zoo/transformer/transformer.go:1276-1287);
    norm = (gain or None, eps, gain_offset) applies RMSNorm first."""
    xn = np.asarray(x, np.float32)
    if norm is not None:
        xn = np_rmsnorm(xn, norm[0], norm[1], norm[2])
    return (np_qdense(t, xn, Wgate, bias_gate, act).astype(np.float64) * np_qdense(t, xn, Wup, bias_up, ACT_NONE).astype(np.float64)).astype(np.float32)


def np_embedding_lookup(t: int, table: np.ndarray, indices: np.ndarray) -> np.ndarray:
    """ggml.EmbeddingLookupDecomposed (ml/ggml/gather.go:21-49); indices [..., 1]."""
    idx = np.asarray(indices)
    if idx.shape[-1] != 1:
        raise ValueError("indices must have last dimension 1")
    flat = idx.reshape(-1).astype(np.int64)
    if flat.size and (flat.min() < 0 or flat.max() >= table.shape[0]):
        raise IndexError("index out of range")
    rows = np_dequantize(t, np.ascontiguousarray(table[flat]))
    return rows.reshape(idx.shape[:-1] + (rows.shape[1],))


# --------------------------------------------------------------------------- C

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build() -> str:
    """Compile libggml_oracle.so with oracle/Makefile (gcc); returns its path."""
    subprocess.run(["make", "-s", "-C", _HERE, "-B"], check=True)
    return os.path.join(_HERE, "libggml_oracle.so")


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libggml_oracle.so")
        if not os.path.exists(path):
            build()
        L = ctypes.CDLL(path)
        vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.gqo_fp16_to_fp32.restype = ctypes.c_float
        L.gqo_fp16_to_fp32.argtypes = [ctypes.c_uint16]
        L.gqo_row_bytes.restype = ctypes.c_size_t
        L.gqo_row_bytes.argtypes = [ci, i64]
        L.gqo_dequantize.argtypes = [ci, vp, i64, i64, vp]
        L.gqo_qdense.argtypes = [ci, vp, i64, i64, vp, i64, vp, ci, vp]
        L.gqo_qdense_f32acc.argtypes = [ci, vp, i64, i64, vp, i64, vp, ci, vp, ci]
        L.gqo_embedding_lookup.argtypes = [ci, vp, i64, i64, vp, i64, vp]
        L.gqo_rmsnorm.argtypes = [vp, i64, i64, vp, ctypes.c_float, ctypes.c_float, vp]
        L.gqo_gated_ffn.argtypes = [ci, vp, i64, i64, ci, vp, ctypes.c_float, ctypes.c_float, vp, vp, vp, vp, i64, ci, vp]
        L.gqo_activation.restype = ctypes.c_float
        L.gqo_activation.argtypes = [ci, ctypes.c_float]
        _LIB = L
    return _LIB


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def c_fp16_to_fp32(h: int) -> float:
    return lib().gqo_fp16_to_fp32(h)


def c_dequantize(t: int, W: np.ndarray, K: int) -> np.ndarray:
    W = np.ascontiguousarray(W, np.uint8)
    out = np.empty((W.shape[0], K), np.float32)
    rc = lib().gqo_dequantize(t, _p(W), W.shape[0], K, _p(out))
    if rc:
        raise ValueError(f"gqo_dequantize failed ({rc})")
    return out


def c_qdense(t: int, x: np.ndarray, W: np.ndarray, bias: np.ndarray | None = None,
             act: int = ACT_NONE, f32acc_threads: int = 0) -> np.ndarray:
    x2 = np.ascontiguousarray(x, np.float32).reshape(-1, x.shape[-1])
    W = np.ascontiguousarray(W, np.uint8)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    M, K = x2.shape
    N = W.shape[0]
    y = np.empty((M, N), np.float32)
    if f32acc_threads:
        rc = lib().gqo_qdense_f32acc(t, _p(x2), M, K, _p(W), N, _p(b), act, _p(y), f32acc_threads)
    else:
        rc = lib().gqo_qdense(t, _p(x2), M, K, _p(W), N, _p(b), act, _p(y))
    if rc:
        raise ValueError(f"gqo_qdense failed ({rc})")
    return y.reshape(x.shape[:-1] + (N,))


def c_embedding_lookup(t: int, table: np.ndarray, K: int, indices: np.ndarray) -> np.ndarray:
    table = np.ascontiguousarray(table, np.uint8)
    idx = np.ascontiguousarray(indices, np.int32).reshape(-1)
    out = np.empty((idx.size, K), np.float32)
    rc = lib().gqo_embedding_lookup(t, _p(table), table.shape[0], K, _p(idx), idx.size, _p(out))
    if rc == -2:
        raise IndexError("index out of range")
    if rc:
        raise ValueError(f"gqo_embedding_lookup failed ({rc})")
    return out.reshape(indices.shape[:-1] + (K,))


def c_rmsnorm(x: np.ndarray, gain: np.ndarray | None = None, eps: float = 1e-6, gain_offset: float = 0.0) -> np.ndarray:
    x2 = np.ascontiguousarray(x, np.float32).reshape(-1, x.shape[-1])
    g = None if gain is None else np.ascontiguousarray(gain, np.float32)
    y = np.empty_like(x2)
    rc = lib().gqo_rmsnorm(_p(x2), x2.shape[0], x2.shape[1], _p(g), eps, gain_offset, _p(y))
    if rc:
        raise ValueError(f"gqo_rmsnorm failed ({rc})")
    return y.reshape(x.shape)


def c_gated_ffn(t: int, x: np.ndarray, Wgate: np.ndarray, Wup: np.ndarray, bias_gate=None, bias_up=None, act: int = ACT_SILU,
                norm: tuple | None = None) -> np.ndarray:
    """norm = (gain or None, eps, gain_offset), or None for no normalisation."""
    x2 = np.ascontiguousarray(x, np.float32).reshape(-1, x.shape[-1])
    Wg, Wu = np.ascontiguousarray(Wgate, np.uint8), np.ascontiguousarray(Wup, np.uint8)
    bg = None if bias_gate is None else np.ascontiguousarray(bias_gate, np.float32)
    bu = None if bias_up is None else np.ascontiguousarray(bias_up, np.float32)
    gain = None if norm is None or norm[0] is None else np.ascontiguousarray(norm[0], np.float32)
    eps, off = (0.0, 0.0) if norm is None else (norm[1], norm[2])
    M, K = x2.shape
    N = Wg.shape[0]
    y = np.empty((M, N), np.float32)
    rc = lib().gqo_gated_ffn(t, _p(x2), M, K, 0 if norm is None else 1, _p(gain), eps, off, _p(Wg), _p(bg), _p(Wu), _p(bu), N, act, _p(y))
    if rc:
        raise ValueError(f"gqo_gated_ffn failed ({rc})")
    return y.reshape(x.shape[:-1] + (N,))
