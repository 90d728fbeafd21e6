"""GGML block formats handled by the quantized Dense path.

Mirrors ``compute.GGMLQuantType`` with its ``BytesPerBlock`` / ``ValuesPerBlock`` methods
(used at ml/ggml/dequant.go:41 and ml/ggml/gather.go:24-25 of the reference) and
``ggml.CanDecompose`` (ml/ggml/dequant.go:20-27).  Numeric values are the public GGML ids.
"""
from __future__ import annotations

Q4_0 = 2
Q8_0 = 8
Q4_K = 12
Q6_K = 14
IQ4_NL = 20

_GEOM = {Q4_0: (18, 32), Q8_0: (34, 32), Q4_K: (144, 256), Q6_K: (210, 256), IQ4_NL: (18, 32)}
_NAMES = {Q4_0: "Q4_0", Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K", IQ4_NL: "IQ4_NL"}


def name(t: int) -> str:
    return _NAMES.get(t, f"GGML({t})")


def bytes_per_block(t: int) -> int:
    return _GEOM[t][0]


def values_per_block(t: int) -> int:
    return _GEOM[t][1]


def row_bytes(t: int, K: int) -> int:
    bpb, vpb = _GEOM[t]
    if K <= 0 or K % vpb:
        raise ValueError(f"K={K} is not a positive multiple of {vpb} for {name(t)}")
    return K // vpb * bpb


def can_decompose(t: int) -> bool:
    """Types with a graph-level decomposed fallback in the reference (ml/ggml/dequant.go:20-27)."""
    return t in (Q4_0, Q8_0, IQ4_NL)
