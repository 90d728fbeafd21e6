"""Pins the CPU oracle (oracle/) before anything is compared against it.

Sources of truth used here, none of which is the oracle's own formula retyped:
  * the reference's known-answer tests (tests/golden/reference_kats.json);
  * IEEE-754 binary16 as implemented by numpy (exhaustive);
  * exact rational arithmetic (fractions.Fraction) rounded once to fp32 for the closed forms
    ml/ggml/dequant.go fixes (Q8_0: f32(d)*f32(q); Q4_0: f32(d)*(nibble-8));
  * structural probes: single non-zero code / scale / min / byte, so that a wrong index,
    nibble order, sign or dropped term fails;
  * the two restatements (numpy, C) against each other on random blocks.
Q4_K and Q6_K have no reference vector (parity unpinned); they get the structural checks only.
"""
import math
import struct
from fractions import Fraction

import numpy as np
import pytest

Q4_0, Q8_0, Q4_K, Q6_K, IQ4_NL = 2, 8, 12, 14, 20
ALL_TYPES = [Q4_0, Q8_0, Q4_K, Q6_K, IQ4_NL]


def f32(x) -> np.float32:
    return np.float32(x)


def round_fraction_to_f32(fr: Fraction) -> np.float32:
    # float(Fraction) rounds correctly to double; all values used here have <= 24 significant
    # bits or are exactly representable in double, so the second rounding is the only one.
    return np.float32(float(fr))


def exact_round_f32(fr: Fraction) -> np.float32:
    """Round-to-nearest-even of an exact rational to binary32, in integer arithmetic (no double in between)."""
    if fr == 0:
        return np.float32(0.0)
    sign, a = (-1, -fr) if fr < 0 else (1, fr)
    n, d = a.numerator, a.denominator
    e = n.bit_length() - d.bit_length()          # 2^e <= a < 2^(e+2), roughly
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -126)                             # below 2^-126 the spacing stays 2^-149
    q = a / Fraction(2) ** (e - 23)              # in units of the last place
    m, rem = divmod(q.numerator, q.denominator)
    twice = 2 * rem
    if twice > q.denominator or (twice == q.denominator and (m & 1)):
        m += 1
    return np.float32(sign * float(m) * float(2.0 ** (e - 23)))   # m < 2^25 and a power of two: exact in double


def is_exact_f32(fr: Fraction) -> bool:
    return Fraction(float(exact_round_f32(fr))) == fr


def half_value(bits: int) -> Fraction:
    """Exact value of a finite binary16 pattern."""
    s = -1 if bits & 0x8000 else 1
    e = (bits >> 10) & 0x1F
    m = bits & 0x3FF
    if e == 0:
        return s * Fraction(m, 1 << 24)
    return s * Fraction((1 << 10) + m, 1 << 10) * Fraction(2) ** (e - 15)


# ------------------------------------------------------------------------------ fp16

def test_fp16_exhaustive_against_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.c_fp16_to_fp32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_fp16_exact_values(oracle):
    for bits in [0x0001, 0x03FF, 0x0400, 0x3C00, 0x7BFF, 0x8001, 0xC000, 0x3555]:
        assert Fraction(float(oracle.c_fp16_to_fp32(bits))) == half_value(bits)


def test_fp16_reference_kats(oracle, kats):
    for k in kats["fp16"]:
        bits = k["bytes"][0] | (k["bytes"][1] << 8)  # little-endian
        assert oracle.c_fp16_to_fp32(bits) == k["value"]
        assert oracle._f16(np.array([k["bytes"]], np.uint8))[0] == k["value"]


# ------------------------------------------------------------------------------ reference KATs

@pytest.mark.parametrize("impl", ["np", "c"])
def test_dense_reference_kats(oracle, kats, impl):
    for k in kats["dense"]:
        W = np.array(k["w"], np.uint8)
        x = np.array(k["x"], np.float32)
        bias = None if k["bias"] is None else np.array(k["bias"], np.float32)
        fn = oracle.np_qdense if impl == "np" else oracle.c_qdense
        got = fn(k["type"], x, W, bias, k["act"])
        assert got.shape == (x.shape[0], W.shape[0])
        np.testing.assert_allclose(got, np.array(k["want"], np.float32), rtol=0, atol=k["tol"], err_msg=k["name"])


@pytest.mark.parametrize("impl", ["np", "c"])
def test_gather_reference_kats(oracle, kats, impl):
    for k in kats["gather"]:
        table = np.array(k["table"], np.uint8)
        idx = np.array(k["indices"], np.int32)
        if impl == "np":
            got = oracle.np_embedding_lookup(k["type"], table, idx)
        else:
            got = oracle.c_embedding_lookup(k["type"], table, 32, idx)
        np.testing.assert_allclose(got, np.array(k["want"], np.float32), rtol=0, atol=k["tol"], err_msg=k["name"])


def test_activation_reference_kats(oracle, kats):
    """ml/layers/activation/activation_test.go:17-112, through both implementations."""
    for k in kats["activation"]:
        x, want = np.array(k["x"], np.float32), np.array(k["want"], np.float32)
        np.testing.assert_allclose(oracle.np_activation(k["act"], x), want, rtol=0, atol=k["tol"], err_msg=k["name"])
        got_c = np.array([oracle.lib().gqo_activation(k["act"], float(v)) for v in x], np.float32)
        np.testing.assert_allclose(got_c, want, rtol=0, atol=k["tol"], err_msg=k["name"])
        if k["tol"] <= 1e-4:  # the published digits are float32-accurate
            np.testing.assert_allclose(got_c, want, rtol=2e-6, atol=2e-7, err_msg=k["name"])


@pytest.mark.parametrize("impl", ["np", "c"])
def test_rmsnorm_reference_kat(oracle, kats, impl):
    """ml/layers/norm/rmsnorm_test.go:16-45: gain of ones (the variable's initial value), default epsilon."""
    fn = oracle.np_rmsnorm if impl == "np" else oracle.c_rmsnorm
    for k in kats["rmsnorm"]:
        x = np.array(k["x"], np.float32)
        for gain in (None, np.ones(x.shape[-1], np.float32)):
            np.testing.assert_allclose(fn(x, gain, k["eps"]), np.array(k["want"], np.float32), rtol=0, atol=k["tol"], err_msg=k["name"])
        # the published digits are good to float32 precision, not just to the test's 1e-3
        np.testing.assert_allclose(fn(x, None, k["eps"]), np.array(k["want"], np.float32), rtol=3e-7, atol=0)


@pytest.mark.parametrize("impl", ["np", "c"])
def test_rmsnorm_closed_forms(oracle, impl):
    fn = oracle.np_rmsnorm if impl == "np" else oracle.c_rmsnorm
    rng = np.random.default_rng(5)
    # a constant row c normalises to sign(c) (eps = 0), times the gain plus its offset
    x = np.full((1, 64), -3.5, np.float32)
    gain = rng.normal(size=64).astype(np.float32)
    np.testing.assert_allclose(fn(x, None, 0.0), -np.ones((1, 64), np.float32), rtol=2e-7)
    np.testing.assert_allclose(fn(x, gain, 0.0, 1.0), -(gain + np.float32(1.0))[None, :], rtol=3e-7)
    # without gain the output has unit mean square; scaling the input by a power of two changes nothing
    x = rng.normal(size=(5, 300)).astype(np.float32)
    y = fn(x, None, 0.0)
    np.testing.assert_allclose(np.mean(y.astype(np.float64) ** 2, axis=-1), 1.0, rtol=1e-6)
    assert np.array_equal(fn(x * np.float32(4.0), None, 0.0), y)
    # a single value with epsilon: x / sqrt(x^2 + eps), here 3 / sqrt(9 + 7) = 0.75
    np.testing.assert_allclose(fn(np.array([[3.0]], np.float32), None, 7.0), [[0.75]], rtol=1e-7)
    # a wrong axis or a sum in place of the mean would fail this: rows are independent
    x2 = np.stack([x[0], 10 * x[0]])
    np.testing.assert_allclose(fn(x2, None, 0.0)[1], fn(x2, None, 0.0)[0], rtol=3e-7)


def test_rmsnorm_c_against_numpy(oracle):
    rng = np.random.default_rng(6)
    x = (rng.normal(size=(7, 4096)) * 3).astype(np.float32)
    gain = rng.normal(size=4096).astype(np.float32)
    np.testing.assert_allclose(oracle.c_rmsnorm(x, gain, 1e-5, 1.0), oracle.np_rmsnorm(x, gain, 1e-5, 1.0), rtol=4e-7, atol=1e-30)


@pytest.mark.parametrize("t", [Q8_0, Q4_K])
def test_gated_ffn_is_the_composition_of_its_parts(oracle, t):
    """activation(dense(xn, Wgate)) * dense(xn, Wup) written out with the pinned pieces."""
    from gomlx_amd import synth
    M, K, N = 3, 512, 24
    Wg, Wu = synth.weights(t, 1, N, K), synth.weights(t, 2, N, K)
    x = synth.activations(3, M, K)
    gain = synth.normal(4, 0, K).astype(np.float32)
    bg, bu = synth.normal(5, 0, N).astype(np.float32), synth.normal(6, 0, N).astype(np.float32)
    for norm in (None, (gain, 1e-6, 1.0), (None, 1e-5, 0.0)):
        xn = x if norm is None else oracle.c_rmsnorm(x, *norm)
        want = oracle.c_qdense(t, xn, Wg, bg, oracle.ACT_SILU).astype(np.float64) * oracle.c_qdense(t, xn, Wu, bu, 0).astype(np.float64)
        got_c = oracle.c_gated_ffn(t, x, Wg, Wu, bg, bu, oracle.ACT_SILU, norm)
        got_np = oracle.np_gated_ffn(t, x, Wg, Wu, bg, bu, oracle.ACT_SILU, norm)
        np.testing.assert_allclose(got_c, want.astype(np.float32), rtol=2e-7, atol=1e-30)
        scale = np.max(np.abs(want))
        assert np.max(np.abs(got_np - want)) / scale < 1e-5
    # swapping the two matrices must change the result (the activation sits on the gate)
    a = oracle.c_gated_ffn(t, x, Wg, Wu, None, None, oracle.ACT_SILU, None)
    b = oracle.c_gated_ffn(t, x, Wu, Wg, None, None, oracle.ACT_SILU, None)
    assert np.max(np.abs(a - b)) > 1e-3 * np.max(np.abs(a))


# ------------------------------------------------------------------------------ closed forms

D_PATTERNS = [0x0000, 0x0001, 0x0155, 0x03FF, 0x0400, 0x1234, 0x2E66, 0x3555, 0x3C00, 0x4000, 0x4200,
              0x5BFF, 0x7BFF, 0x8400, 0xBC00, 0xFBFF]


@pytest.mark.parametrize("impl", ["np", "c"])
def test_q8_0_closed_form_all_codes(oracle, impl):
    # one block per row; code byte i of row r is (r + 8*i) mod 256, so all 256 codes appear
    # in every position class across rows
    for dbits in D_PATTERNS:
        W = np.zeros((256, 34), np.uint8)
        W[:, 0], W[:, 1] = dbits & 0xFF, dbits >> 8
        codes = (np.arange(256)[:, None] + 8 * np.arange(32)[None, :]) % 256
        W[:, 2:] = codes
        got = oracle.np_dequantize(Q8_0, W) if impl == "np" else oracle.c_dequantize(Q8_0, W, 32)
        d = half_value(dbits)
        for r in range(0, 256, 17):
            for i in range(32):
                q = int(codes[r, i])
                q = q - 256 if q >= 128 else q
                want = round_fraction_to_f32(d * q)
                assert got[r, i] == want, (hex(dbits), r, i)


@pytest.mark.parametrize("impl", ["np", "c"])
def test_q4_0_closed_form_and_nibble_order(oracle, impl):
    # ml/ggml/dequant.go:94-96: value j (<16) is the LOW nibble of byte j, value 16+j the HIGH nibble.
    rng = np.random.default_rng(5)
    for dbits in D_PATTERNS:
        W = rng.integers(0, 256, size=(8, 18), dtype=np.uint8)
        W[:, 0], W[:, 1] = dbits & 0xFF, dbits >> 8
        got = oracle.np_dequantize(Q4_0, W) if impl == "np" else oracle.c_dequantize(Q4_0, W, 32)
        d = half_value(dbits)
        for r in range(8):
            for j in range(16):
                b = int(W[r, 2 + j])
                assert got[r, j] == round_fraction_to_f32(d * ((b & 15) - 8))
                assert got[r, 16 + j] == round_fraction_to_f32(d * ((b >> 4) - 8))


IQ4NL_PUBLIC = [-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113]


@pytest.mark.parametrize("impl", ["np", "c"])
def test_iq4_nl_table_and_order(oracle, impl):
    W = np.zeros((16, 18), np.uint8)
    W[:, 1] = 0x3C  # d = 1.0
    for n in range(16):
        W[n, 2:] = 0x88
        W[n, 2 + 3] = n | ((15 - n) << 4)  # low nibble n at value 3, high nibble 15-n at value 19
    got = oracle.np_dequantize(IQ4_NL, W) if impl == "np" else oracle.c_dequantize(IQ4_NL, W, 32)
    for n in range(16):
        assert got[n, 3] == IQ4NL_PUBLIC[n]
        assert got[n, 19] == IQ4NL_PUBLIC[15 - n]
        assert got[n, 0] == 1.0  # LUT[8], ml/nn/quantized_dense_test.go:409
    assert IQ4NL_PUBLIC[9] == 13


# ------------------------------------------------------------------------------ Q4_K structure

def pack_q4k_scales(sc, mn):
    """Inverse of the 6-bit unpacking, written from the public GGML layout: bytes 0-3 hold
    sc[0..3] (low 6 bits) + high 2 bits of sc[4..7]; bytes 4-7 hold mn[0..3] + high 2 bits of
    mn[4..7]; bytes 8-11 hold low nibbles of sc[4..7] | low nibbles of mn[4..7] << 4."""
    s = [0] * 12
    for j in range(4):
        s[j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        s[j + 4] = (mn[j] & 63) | ((mn[j + 4] >> 4) << 6)
        s[j + 8] = (sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)
    return s


def make_q4k_block(dbits, dminbits, sc, mn, codes):
    """codes: 256 ints in [0,15] in logical order."""
    b = np.zeros(144, np.uint8)
    b[0], b[1], b[2], b[3] = dbits & 0xFF, dbits >> 8, dminbits & 0xFF, dminbits >> 8
    b[4:16] = pack_q4k_scales(sc, mn)
    for g in range(4):
        for l in range(32):
            b[16 + 32 * g + l] = codes[64 * g + l] | (codes[64 * g + 32 + l] << 4)
    return b


@pytest.mark.parametrize("impl", ["np", "c"])
def test_q4_k_full_block_against_exact_arithmetic(oracle, impl):
    rng = np.random.default_rng(11)
    for trial in range(6):
        sc = [int(v) for v in rng.integers(0, 64, 8)]
        mn = [int(v) for v in rng.integers(0, 64, 8)]
        codes = [int(v) for v in rng.integers(0, 16, 256)]
        dbits, dminbits = [0x2E66, 0x1A00, 0x0155, 0x3C00, 0x0001, 0x3555][trial], [0x2A00, 0x0003, 0x1234, 0x3800, 0x0400, 0x2101][trial]
        W = make_q4k_block(dbits, dminbits, sc, mn, codes)[None, :]
        got = oracle.np_dequantize(Q4_K, W) if impl == "np" else oracle.c_dequantize(Q4_K, W, 256)
        d, dmin = half_value(dbits), half_value(dminbits)
        for i in range(256):
            j = i // 32
            ds = round_fraction_to_f32(d * sc[j])            # (d * sc)      rounded
            dm = round_fraction_to_f32(dmin * mn[j])         # (dmin * m)    rounded
            prod = round_fraction_to_f32(Fraction(float(ds)) * codes[i])   # ds * q rounded
            want = round_fraction_to_f32(Fraction(float(prod)) - Fraction(float(dm)))
            assert got[0, i] == want, (trial, i)


@pytest.mark.parametrize("impl", ["np", "c"])
def test_q4_k_value_is_one_correctly_rounded_subtraction(oracle, impl):
    """w = d*sc*q - dmin*m needs ONE rounding whatever the order of operations: d*sc (11 + 6 bits), (d*sc)*q and d*(sc*q)
    (<= 21 bits) and dmin*m (<= 17 bits) are all exact in binary32, so every association of the products, with or
    without a fused multiply-add for the subtraction, yields fl(d*sc*q - dmin*m).  The oracle is compared with that
    closed form, rounded once from exact rationals; what this leaves open about the external Go code is the byte layout
    alone, not its arithmetic."""
    rng = np.random.default_rng(2024)
    dpats = [0x0001, 0x0155, 0x03FF, 0x0400, 0x1A00, 0x2E66, 0x3555, 0x3C00, 0x3FFF, 0x7BFF, 0x4D2B, 0x12AB]
    for trial in range(40):
        dbits, dminbits = dpats[trial % len(dpats)], dpats[(5 * trial + 3) % len(dpats)]
        if trial >= 24:
            dbits, dminbits = int(rng.integers(1, 0x7C00)), int(rng.integers(1, 0x7C00))
        sc = [int(v) for v in rng.integers(0, 64, 8)]
        mn = [int(v) for v in rng.integers(0, 64, 8)]
        sc[0], mn[0], sc[1], mn[1] = 63, 63, 63, 0
        codes = [int(v) for v in rng.integers(0, 16, 256)]
        codes[0], codes[1], codes[32] = 15, 0, 15
        W = make_q4k_block(dbits, dminbits, sc, mn, codes)[None, :]
        got = oracle.np_dequantize(Q4_K, W) if impl == "np" else oracle.c_dequantize(Q4_K, W, 256)
        d, dmin = half_value(dbits), half_value(dminbits)
        for i in range(256):
            j, q = i // 32, codes[i]
            # every intermediate product is a binary32 number: no association of the multiplications rounds
            assert is_exact_f32(d * sc[j]) and is_exact_f32(d * sc[j] * q) and is_exact_f32(d * (sc[j] * q)) and is_exact_f32(dmin * mn[j])
            want = exact_round_f32(d * sc[j] * q - dmin * mn[j])
            assert got[0, i] == want, (trial, i, dbits, dminbits)


def test_exact_rounding_helper():
    for v in (Fraction(1, 3), Fraction(-7, 5), Fraction(1, 1 << 140), Fraction(3, 1 << 149), Fraction((1 << 24) + 1, 1), Fraction((1 << 25) + 2, 3),
              Fraction(16777215, 1 << 150), Fraction(1, 1 << 150)):
        assert exact_round_f32(v) == np.float32(float(v)), v   # (doubles are exact or far from a tie for these)
    assert exact_round_f32(Fraction((1 << 24) + 1, 1)) == np.float32(16777216.0)       # tie to even
    assert exact_round_f32(Fraction((1 << 24) + 3, 1)) == np.float32(16777220.0)
    assert exact_round_f32(Fraction(1, 1 << 150)) == np.float32(0.0)                   # half the smallest subnormal: tie to even


@pytest.mark.parametrize("impl", ["np", "c"])
def test_q4_k_single_field_probes(oracle, impl):
    deq = (lambda W: oracle.np_dequantize(Q4_K, W)) if impl == "np" else (lambda W: oracle.c_dequantize(Q4_K, W, 256))
    # (a) one sub-block scale, all codes 1: exactly that sub-block's 32 values light up
    for j in range(8):
        sc = [0] * 8
        sc[j] = 37 + j
        W = make_q4k_block(0x3C00, 0x3C00, sc, [0] * 8, [1] * 256)[None, :]
        out = deq(W)[0]
        want = np.zeros(256, np.float32)
        want[32 * j:32 * j + 32] = 37 + j
        assert np.array_equal(out, want), j
    # (b) one sub-block min: that sub-block is shifted down by dmin*m, codes irrelevant (0)
    for j in range(8):
        mn = [0] * 8
        mn[j] = 63 - j
        W = make_q4k_block(0x3C00, 0x4000, [0] * 8, mn, [0] * 256)[None, :]
        out = deq(W)[0]
        want = np.zeros(256, np.float32)
        want[32 * j:32 * j + 32] = -2.0 * (63 - j)
        assert np.array_equal(out, want), j
    # (c) one code: exactly one value
    for i in [0, 1, 31, 32, 33, 63, 64, 100, 191, 192, 224, 255]:
        codes = [0] * 256
        codes[i] = 11
        W = make_q4k_block(0x3C00, 0x0000, [1] * 8, [0] * 8, codes)[None, :]
        out = deq(W)[0]
        want = np.zeros(256, np.float32)
        want[i] = 11.0
        assert np.array_equal(out, want), i


def test_q4_k_byte_footprint(oracle):
    """Flipping code byte b of a super-block changes exactly the two values the layout assigns to it."""
    rng = np.random.default_rng(3)
    base = make_q4k_block(0x3C00, 0x3800, [int(v) for v in rng.integers(1, 64, 8)],
                          [int(v) for v in rng.integers(0, 64, 8)], [int(v) for v in rng.integers(0, 16, 256)])
    ref = oracle.c_dequantize(Q4_K, base[None, :], 256)[0]
    for b in range(128):
        mod = base.copy()
        mod[16 + b] ^= 0xFF
        out = oracle.c_dequantize(Q4_K, mod[None, :], 256)[0]
        changed = set(np.nonzero(out != ref)[0].tolist())
        g, l = divmod(b, 32)
        assert changed == {64 * g + l, 64 * g + 32 + l}, b


# ------------------------------------------------------------------------------ Q6_K structure

def make_q6k_block(dbits, scales, codes):
    """codes: 256 ints in [0,63] in logical order; scales: 16 ints in [-128,127].  Written from the
    public GGML layout: for half h and l = 0..31 the values 128h + l, + 32 + l, + 64 + l, + 96 + l
    share byte 32h + l of qh (2 bits each, low to high) and use the low / high nibbles of
    ql[64h + l] and ql[64h + 32 + l]."""
    b = np.zeros(210, np.uint8)
    for h in range(2):
        for l in range(32):
            q = [codes[128 * h + 32 * k + l] for k in range(4)]
            b[64 * h + l] = (q[0] & 15) | ((q[2] & 15) << 4)
            b[64 * h + 32 + l] = (q[1] & 15) | ((q[3] & 15) << 4)
            b[128 + 32 * h + l] = (q[0] >> 4) | ((q[1] >> 4) << 2) | ((q[2] >> 4) << 4) | ((q[3] >> 4) << 6)
    for j in range(16):
        b[192 + j] = scales[j] & 0xFF
    b[208], b[209] = dbits & 0xFF, dbits >> 8
    return b


@pytest.mark.parametrize("impl", ["np", "c"])
def test_q6_k_full_block_against_exact_arithmetic(oracle, impl):
    """w = d * scale * (q - 32) is exactly representable in fp32 (11 + 7 + 6 bits), so the expected
    value is the exact rational product."""
    rng = np.random.default_rng(17)
    for trial, dbits in enumerate([0x2E66, 0x1A00, 0x3C00, 0x0155, 0x3555, 0xAE66]):
        scales = [int(v) for v in rng.integers(-128, 128, 16)]
        codes = [int(v) for v in rng.integers(0, 64, 256)]
        W = make_q6k_block(dbits, scales, codes)[None, :]
        got = oracle.np_dequantize(Q6_K, W) if impl == "np" else oracle.c_dequantize(Q6_K, W, 256)
        d = half_value(dbits)
        for i in range(256):
            want = d * scales[i // 16] * (codes[i] - 32)
            assert Fraction(float(got[0, i])) == want, (trial, i)


@pytest.mark.parametrize("impl", ["np", "c"])
def test_q6_k_single_field_probes(oracle, impl):
    deq = (lambda W: oracle.np_dequantize(Q6_K, W)) if impl == "np" else (lambda W: oracle.c_dequantize(Q6_K, W, 256))
    # (a) one scale, all codes 33 (q - 32 = 1): exactly that scale's 16 values light up
    for j in range(16):
        scales = [0] * 16
        scales[j] = 5 + j if j % 2 else -(5 + j)
        out = deq(make_q6k_block(0x3C00, scales, [33] * 256)[None, :])[0]
        want = np.zeros(256, np.float32)
        want[16 * j:16 * j + 16] = scales[j]
        assert np.array_equal(out, want), j
    # (b) one code: exactly one value, over the whole 6-bit range incl. the high two bits
    for i, c in [(0, 63), (1, 0), (31, 47), (32, 16), (95, 32 + 17), (96, 1), (127, 62), (128, 63), (200, 48), (255, 15)]:
        codes = [32] * 256
        codes[i] = c
        out = deq(make_q6k_block(0x4000, [1] * 16, codes)[None, :])[0]
        want = np.zeros(256, np.float32)
        want[i] = 2.0 * (c - 32)
        assert np.array_equal(out, want), (i, c)


def test_q6_k_byte_footprint(oracle):
    """Flipping a byte of ql changes exactly two values, a byte of qh exactly four, a scale sixteen."""
    rng = np.random.default_rng(5)
    codes = [int(v) if v != 32 else 7 for v in rng.integers(0, 64, 256)]  # code 32 decodes to 0 whatever the scale
    base = make_q6k_block(0x3C00, [int(v) for v in rng.integers(1, 100, 16)], codes)
    ref = oracle.c_dequantize(Q6_K, base[None, :], 256)[0]

    def changed(byte):
        mod = base.copy()
        mod[byte] ^= 0xFF
        return set(np.nonzero(oracle.c_dequantize(Q6_K, mod[None, :], 256)[0] != ref)[0].tolist())

    for b in range(128):
        h, r = divmod(b, 64)
        which, l = divmod(r, 32)
        assert changed(b) == {128 * h + 32 * which + l, 128 * h + 64 + 32 * which + l}, b
    for b in range(64):
        h, l = divmod(b, 32)
        assert changed(128 + b) == {128 * h + 32 * k + l for k in range(4)}, b
    for j in range(16):
        assert changed(192 + j) == set(range(16 * j, 16 * j + 16)), j


# ------------------------------------------------------------------------------ numpy vs C

def random_blocks(t, N, K, seed):
    from gomlx_amd import synth
    return synth.weights(t, seed, N, K)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_numpy_and_c_agree_bit_exactly_on_dequant(oracle, t):
    K = 512
    W = random_blocks(t, 37, K, 100 + t)
    a = oracle.np_dequantize(t, W, K)
    b = oracle.c_dequantize(t, W, K)
    assert a.dtype == b.dtype == np.float32 and a.shape == b.shape == (37, K)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("t", ALL_TYPES)
def test_numpy_and_c_agree_on_dense(oracle, t):
    from gomlx_amd import synth
    K, N, M = 768, 33, 5
    W = random_blocks(t, N, K, 200 + t)
    x = synth.activations(300 + t, M, K)
    bias = synth.normal(400 + t, 0, N).astype(np.float32)
    for act in range(6):
        a = oracle.np_qdense(t, x, W, bias, act)
        b = oracle.c_qdense(t, x, W, bias, act)
        np.testing.assert_allclose(a, b, rtol=2e-6, atol=1e-7)
    c = oracle.c_qdense(t, x, W, bias, 0, f32acc_threads=3)
    gold = oracle.c_qdense(t, x, W, bias, 0)
    assert np.max(np.abs(c - gold)) <= 1e-5 * np.max(np.abs(gold))


# ------------------------------------------------------------------------------ dense invariants

@pytest.mark.parametrize("t", ALL_TYPES)
def test_dense_unit_vectors_return_columns_exactly(oracle, t):
    K, N = 256, 9
    W = random_blocks(t, N, K, 500 + t)
    Wd = oracle.c_dequantize(t, W, K)
    for k in [0, 1, 15, 16, 31, 32, 100, 255]:
        x = np.zeros((1, K), np.float32)
        x[0, k] = 1.0
        y = oracle.c_qdense(t, x, W)
        assert np.array_equal(y[0], Wd[:, k]), k


@pytest.mark.parametrize("t", ALL_TYPES)
def test_dense_linearity_bias_and_row_permutation(oracle, t):
    from gomlx_amd import synth
    K, N = 512, 12
    W = random_blocks(t, N, K, 600 + t)
    x = synth.activations(601, 2, K)
    y = oracle.c_qdense(t, x, W)
    y_sum = oracle.c_qdense(t, (x[0] + 2.0 * x[1])[None, :].astype(np.float32), W)
    np.testing.assert_allclose(y_sum[0], y[0] + 2.0 * y[1], rtol=1e-5, atol=1e-6)
    bias = np.arange(N, dtype=np.float32)
    assert np.array_equal(oracle.c_qdense(t, np.zeros((1, K), np.float32), W, bias)[0], bias)
    perm = np.random.default_rng(0).permutation(N)
    assert np.array_equal(oracle.c_qdense(t, x, W[perm]), y[:, perm])


def test_dense_leading_batch_axes(oracle):
    from gomlx_amd import synth
    W = random_blocks(Q8_0, 7, 64, 1)
    x = synth.activations(2, 6, 64).reshape(2, 3, 64)
    y = oracle.np_qdense(Q8_0, x, W)
    assert y.shape == (2, 3, 7)
    assert np.array_equal(y.reshape(6, 7), oracle.np_qdense(Q8_0, x.reshape(6, 64), W))


# ------------------------------------------------------------------------------ epilogue

def test_activation_formulas(oracle):
    xs = [-7.5, -3.0, -1.0, -0.25, 0.0, 0.3, 1.0, 2.0, 3.0, 6.5]
    for x in xs:
        want = {
            0: x,
            1: x * 0.5 * (1.0 + math.erf(x / math.sqrt(2.0))),          # activation.go:274-286
            2: max(x, 0.0),                                             # activation.go:161
            3: x / (1.0 + math.exp(-x)),                                # activation.go:195
            4: x * min(max(x / 6.0 + 0.5, 0.0), 1.0),                   # activation.go:222-243
            5: math.tanh(x),
        }
        for act, w in want.items():
            assert abs(oracle.lib().gqo_activation(act, x) - w) <= 1e-6 * max(1.0, abs(w)), (act, x)
            assert abs(float(oracle.np_activation(act, np.array([x], np.float32))[0]) - w) <= 1e-6 * max(1.0, abs(w))
    # SiLU values quoted by the reference test (ml/nn/quantized_dense_test.go:394-398)
    assert abs(oracle.lib().gqo_activation(3, 2.0) - 1.7616) < 1e-3
    assert abs(oracle.lib().gqo_activation(3, 3.0) - 2.8577) < 1e-3


# ------------------------------------------------------------------------------ error behaviour

def test_oracle_rejects_ragged_and_unknown(oracle):
    W = np.zeros((2, 35), np.uint8)
    with pytest.raises(ValueError):
        oracle.np_dequantize(Q8_0, W)
    with pytest.raises(ValueError):
        oracle.c_dequantize(Q8_0, np.zeros((2, 34), np.uint8), 33)
    with pytest.raises(ValueError):
        oracle.c_dequantize(99, np.zeros((2, 34), np.uint8), 32)
    assert oracle.row_bytes(Q4_K, 255) == 0 and oracle.lib().gqo_row_bytes(Q4_K, 255) == 0
    assert oracle.row_bytes(Q4_K, 14336) == 8064 == oracle.lib().gqo_row_bytes(Q4_K, 14336)
    assert oracle.row_bytes(Q6_K, 14336) == 11760 == oracle.lib().gqo_row_bytes(Q6_K, 14336)
    assert oracle.row_bytes(Q8_0, 4096) == 4352 and oracle.row_bytes(Q4_0, 4096) == 2304


def test_gather_index_errors_and_empty(oracle):
    table = random_blocks(Q4_0, 5, 64, 9)
    with pytest.raises(IndexError):
        oracle.c_embedding_lookup(Q4_0, table, 64, np.array([[5]], np.int32))
    with pytest.raises(IndexError):
        oracle.np_embedding_lookup(Q4_0, table, np.array([[-1]], np.int32))
    out = oracle.c_embedding_lookup(Q4_0, table, 64, np.zeros((0, 1), np.int32))
    assert out.shape == (0, 64)
    idx = np.array([[[4], [0]], [[2], [2]]], np.int32)
    got = oracle.np_embedding_lookup(Q4_0, table, idx)
    assert got.shape == (2, 2, 64)
    assert np.array_equal(got.reshape(4, 64), oracle.c_dequantize(Q4_0, table, 64)[[4, 0, 2, 2]])
