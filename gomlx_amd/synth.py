"""Seeded synthetic GGML weights and activations for the benchmark configurations.

A counter-based generator (splitmix64 finaliser over ``seed`` and the element index) so
any slice of a tensor can be regenerated independently and the bytes do not depend on
numpy's own bit generators.  Streams: one per (seed, stream-id) pair.
"""
from __future__ import annotations

import numpy as np

from . import ggml

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def _mix(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def bits64(seed: int, stream: int, n: int, offset: int = 0) -> np.ndarray:
    """n 64-bit words of stream (seed, stream), starting at element ``offset``."""
    with np.errstate(over="ignore"):
        base = _mix(np.uint64(seed) * _GOLDEN + np.uint64(stream) + np.uint64(1))
        idx = np.arange(offset, offset + n, dtype=np.uint64)
        return _mix(base + (idx + np.uint64(1)) * _GOLDEN)


def uniform(seed: int, stream: int, n: int) -> np.ndarray:
    """float64 uniform in (0, 1)."""
    return ((bits64(seed, stream, n) >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / (1 << 53))


def normal(seed: int, stream: int, n: int) -> np.ndarray:
    """float64 N(0,1) by Box-Muller (cosine branch) on two sub-streams."""
    u1 = uniform(seed, 2 * stream + 1000, n)
    u2 = uniform(seed, 2 * stream + 1001, n)
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)


def randint(seed: int, stream: int, n: int, lo: int, hi: int) -> np.ndarray:
    """int64 uniform on the closed range [lo, hi]."""
    span = np.uint64(hi - lo + 1)
    return ((bits64(seed, stream, n) >> np.uint64(16)) % span).astype(np.int64) + lo


def activations(seed: int, M: int, K: int, dtype=np.float32) -> np.ndarray:
    """x ~ N(0,1), [M, K]."""
    return normal(seed, 7, M * K).reshape(M, K).astype(dtype)


def _f16_bytes(v: np.ndarray) -> np.ndarray:
    return v.astype(np.float16).view(np.uint8).reshape(v.shape + (2,))


def weights(ggml_type: int, seed: int, N: int, K: int) -> np.ndarray:
    """Random GGML blocks, [N, row_bytes] uint8, distributed as the benchmark configs state.

    Q8_0: d = fp16(|N(0,0.02)|/127), q uniform in [-127,127].
    Q4_0 / IQ4_NL: d = fp16(|N(0,0.02)|/8), nibbles uniform in [0,15].
    Q4_K: d = fp16(|N(0,0.002)|), dmin = fp16(|N(0,0.001)|), 6-bit scales/mins uniform in
    [0,63] (so all 12 packed bytes are uniform), codes uniform in [0,15].
    """
    bpb, vpb = ggml.bytes_per_block(ggml_type), ggml.values_per_block(ggml_type)
    if K % vpb:
        raise ValueError("K must be a whole number of blocks")
    nb = N * (K // vpb)
    out = np.empty((nb, bpb), np.uint8)
    if ggml_type == ggml.Q8_0:
        out[:, 0:2] = _f16_bytes(np.abs(normal(seed, 1, nb)) * 0.02 / 127.0)
        q = randint(seed, 2, nb * 32, -127, 127).astype(np.int8)
        out[:, 2:34] = q.view(np.uint8).reshape(nb, 32)
    elif ggml_type in (ggml.Q4_0, ggml.IQ4_NL):
        out[:, 0:2] = _f16_bytes(np.abs(normal(seed, 1, nb)) * 0.02 / 8.0)
        out[:, 2:18] = (bits64(seed, 2, nb * 16) >> np.uint64(24)).astype(np.uint8).reshape(nb, 16)
    elif ggml_type == ggml.Q4_K:
        out[:, 0:2] = _f16_bytes(np.abs(normal(seed, 1, nb)) * 0.002)
        out[:, 2:4] = _f16_bytes(np.abs(normal(seed, 3, nb)) * 0.001)
        out[:, 4:16] = (bits64(seed, 4, nb * 12) >> np.uint64(24)).astype(np.uint8).reshape(nb, 12)
        out[:, 16:144] = (bits64(seed, 2, nb * 128) >> np.uint64(24)).astype(np.uint8).reshape(nb, 128)
    elif ggml_type == ggml.Q6_K:  # d = fp16(|N(0, 2e-5)|), int8 scales and all code bits uniform
        out[:, 0:192] = (bits64(seed, 2, nb * 192) >> np.uint64(24)).astype(np.uint8).reshape(nb, 192)
        out[:, 192:208] = (bits64(seed, 4, nb * 16) >> np.uint64(24)).astype(np.uint8).reshape(nb, 16)
        out[:, 208:210] = _f16_bytes(np.abs(normal(seed, 1, nb)) * 2e-5)
    else:
        raise ValueError(f"unsupported ggml type {ggml_type}")
    return out.reshape(N, (K // vpb) * bpb)
