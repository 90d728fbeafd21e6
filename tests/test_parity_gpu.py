"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on identical inputs.

Bars (from the task statement): dequantised weights bit-exact; fp32-activation outputs within
1e-3, bf16-MFMA outputs within 2e-2, both measured as max|got - want| / max|want| over the
output (per-element relative error is meaningless for near-cancelling sums of thousands of
N(0,1) terms).
"""
import numpy as np
import pytest

from gomlx_amd import ggml, nn, synth
from gomlx_amd.nn import Activation, Quantization

pytestmark = pytest.mark.gpu

Q4_0, Q8_0, Q4_K, Q6_K, IQ4_NL = ggml.Q4_0, ggml.Q8_0, ggml.Q4_K, ggml.Q6_K, ggml.IQ4_NL
ALL_TYPES = [Q4_0, Q8_0, Q4_K, Q6_K, IQ4_NL]
TOL_F32 = 1e-3
TOL_BF16 = 2e-2

BACKEND_ACT = {0: Activation.NONE, 1: Activation.GELU, 2: Activation.RELU, 3: Activation.SILU,
               4: Activation.HARD_SWISH, 5: Activation.TANH}


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


# test name -> [worst max|d| / max|want|, worst max|d| / rms(want)] over every comparison the test made; printed at the end
# of the session (tests/conftest.py) so that the margin to the bounds is visible per kernel family.
MARGINS = {}


def rms_err(got, want):
    """The per-element form of the bound: the largest |got - want| over rms(want) (|d| <= tol * rms(want) for every element)."""
    rms = float(np.sqrt(np.mean(np.square(want.astype(np.float64))))) or 1.0
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) / rms


def rel_err(got, want):
    import os
    scale = float(np.max(np.abs(want))) or 1.0
    err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) / scale
    key = os.environ.get("PYTEST_CURRENT_TEST", "?").split("::")[-1].split(" ")[0].split("[")[0]
    rec = MARGINS.setdefault(key, [0.0, 0.0])
    rec[0], rec[1] = max(rec[0], err), max(rec[1], rms_err(got, want))
    return err


def run_dense(torch, t, x, W, bias=None, act=0, bf16=False):
    xd = dev(torch, x)
    if bf16:
        xd = xd.to(torch.bfloat16)
    y = nn.quantized_dense(xd, dev(torch, W), Quantization(ggml_type=t), None if bias is None else dev(torch, bias),
                           BACKEND_ACT[act])
    torch.cuda.synchronize()
    return y.cpu().numpy()


def bf16_round(x):
    import torch
    return torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()


# ------------------------------------------------------------------------------ reference KATs

def test_reference_dense_kats(gpu, kats):
    for k in kats["dense"]:
        got = run_dense(gpu, k["type"], np.array(k["x"], np.float32), np.array(k["w"], np.uint8),
                        None if k["bias"] is None else np.array(k["bias"], np.float32), k["act"])
        np.testing.assert_allclose(got, np.array(k["want"], np.float32), rtol=0, atol=k["tol"], err_msg=k["name"])


def test_reference_gather_kats(gpu, kats):
    for k in kats["gather"]:
        out = nn.quantized_gather(dev(gpu, np.array(k["table"], np.uint8)), dev(gpu, np.array(k["indices"], np.int32)),
                                  Quantization(ggml_type=k["type"]))
        np.testing.assert_allclose(out.cpu().numpy(), np.array(k["want"], np.float32), rtol=0, atol=k["tol"],
                                   err_msg=k["name"])


def test_reference_activation_kats(gpu, kats):
    """The reference's activation vectors (ml/layers/activation/activation_test.go:17-112) through the
    fused epilogue: a Q8_0 identity matrix (scale 1.0, code 1 on the diagonal) hands x to the activation
    unchanged, at one row (decode GEMV) and at 40 rows (MFMA path)."""
    K = 32
    W = np.zeros((7, 34), np.uint8)
    W[:, 1] = 0x3C  # fp16 1.0, little-endian
    for i in range(7):
        W[i, 2 + i] = 1
    for k in kats["activation"]:
        x = np.zeros((1, K), np.float32)
        x[0, :7] = k["x"]
        for rows in (1, 40):
            got = run_dense(gpu, Q8_0, np.repeat(x, rows, axis=0), W, None, k["act"])
            np.testing.assert_allclose(got, np.repeat(np.array([k["want"]], np.float32), rows, axis=0), rtol=0, atol=k["tol"],
                                       err_msg=k["name"])


# ------------------------------------------------------------------------------ dequantisation (bit-exact)

@pytest.mark.parametrize("t", ALL_TYPES)
@pytest.mark.parametrize("N,K", [(1, 256), (37, 512), (300, 4096)])
def test_dequantize_bit_exact(gpu, oracle, t, N, K):
    W = synth.weights(t, 10 + t, N, K)
    got = nn.dequantize(dev(gpu, W), t).cpu().numpy()
    want = oracle.c_dequantize(t, W, K)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("t", ALL_TYPES)
def test_dequantize_bit_exact_on_extreme_scales(gpu, oracle, t):
    """Random bytes everywhere, including the fp16 scale fields (subnormals, large values)."""
    K, N = 1024, 64
    rb = ggml.row_bytes(t, K)
    raw = (synth.bits64(77, t, N * rb) >> np.uint64(20)).astype(np.uint8).reshape(N, rb)
    blk = raw.reshape(N, -1, ggml.bytes_per_block(t))
    # keep the fp16 fields finite (exponent != 31): inf/NaN scales are outside the contract
    for off in {Q4_K: [1, 3], Q6_K: [209]}.get(t, [1]):
        hi = blk[:, :, off]
        hi[(hi & 0x7C) == 0x7C] &= 0xBF
    got = nn.dequantize(dev(gpu, raw), t).cpu().numpy()
    want = oracle.c_dequantize(t, raw, K)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequantize_full_size_config0(gpu, oracle):
    W = synth.weights(Q8_0, 1000, 4096, 4096)
    got = nn.dequantize(dev(gpu, W), Q8_0).cpu().numpy()
    want = oracle.c_dequantize(Q8_0, W, 4096)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# ------------------------------------------------------------------------------ decode GEMV (fp32)

@pytest.mark.parametrize("t", ALL_TYPES)
@pytest.mark.parametrize("M,K,N", [(1, 256, 1), (1, 512, 7), (2, 1024, 33), (3, 4096, 130), (4, 2048, 257), (1, 14336, 64)])
def test_gemv_parity(gpu, oracle, t, M, K, N):
    W = synth.weights(t, 20 + t, N, K)
    x = synth.activations(21 + t, M, K)
    bias = synth.normal(22 + t, 0, N).astype(np.float32) * 0.1
    for act in (0, 3):
        got = run_dense(gpu, t, x, W, bias, act)
        want = oracle.c_qdense(t, x, W, bias, act)
        assert got.shape == (M, N)
        assert rel_err(got, want) < TOL_F32, (t, M, K, N, act)


@pytest.mark.parametrize("t", [Q4_0, Q8_0, Q4_K, Q6_K, IQ4_NL])
@pytest.mark.parametrize("M,K,N", [
    (1, 1536, 100),     # 3 slices of 512: three wavefronts per workgroup
    (2, 3584, 513),     # 7 slices, rows not a multiple of 8
    (1, 4608, 40),      # 9 slices on 8 wavefronts: the first takes two
    (2, 256, 33),       # a single half slice
    (1, 768, 100),      # one slice and a half
    (3, 5376, 50),      # ten slices and a half: uneven shares and a half tail
    (1, 9472, 300),     # eighteen and a half
    (1, 18944, 24),     # 37 slices (a prime): 5 or 4 per wavefront
    (1, 8192, 2100),    # two slices per wavefront
    (3, 2048, 20000),   # five row-steps per wavefront, all in flight
    (1, 512, 300000),   # one wavefront per workgroup, many groups of four row-steps
    (1, 8192, 40000),   # groups of four row-steps wrapping from one slice to the next
])
def test_gemv_k_sliced_plans(gpu, oracle, t, M, K, N):
    """Shapes that walk through the planner of the K-sliced decode kernel: wavefronts per
    workgroup, even and uneven slices per wavefront, a last half slice, prefetch groups."""
    W = synth.weights(t, 40 + t, N, K)
    x = synth.activations(41 + t, M, K)
    bias = synth.normal(42 + t, 0, N).astype(np.float32) * 0.1
    got = run_dense(gpu, t, x, W, bias, 0)
    want = oracle.c_qdense(t, x, W, bias, 0)
    assert got.shape == (M, N)
    assert rel_err(got, want) < TOL_F32, (t, M, K, N)


@pytest.mark.parametrize("t", [Q4_0, Q8_0, Q4_K, Q6_K, IQ4_NL])
@pytest.mark.parametrize("M,K,N", [(1, 4096, 300), (3, 1024, 257), (16, 2048, 130)])
def test_bf16_decode_batches_are_exact_widenings(gpu, oracle, t, M, K, N):
    """bf16 activations of a decode batch run through the fp32 GEMV (bf16 -> fp32 is exact), so
    they meet the fp32 tolerance against the oracle on the same bf16-valued inputs."""
    W = synth.weights(t, 50 + t, N, K)
    x = bf16_round(synth.activations(51 + t, M, K))
    bias = synth.normal(52 + t, 0, N).astype(np.float32) * 0.1
    got = run_dense(gpu, t, x, W, bias, 3, bf16=True)
    assert rel_err(got, oracle.c_qdense(t, x, W, bias, 3)) < TOL_F32, (t, M, K, N)


@pytest.mark.parametrize("t", [Q4_0, Q8_0, Q6_K, IQ4_NL])
@pytest.mark.parametrize("M", [5, 9, 16, 17])
def test_small_batches_f32(gpu, oracle, t, M):
    """Batches just above the decode sizes: GEMV passes up to 16 rows where the format has no
    small-batch MFMA kernel, the tiled kernel beyond (and for IQ4_NL)."""
    K, N = 1024, 300
    W = synth.weights(t, 60 + t, N, K)
    x = synth.activations(61 + t, M, K)
    got = run_dense(gpu, t, x, W, None, 0)
    assert rel_err(got, oracle.c_qdense(t, x, W, None, 0)) < TOL_F32, (t, M)


@pytest.mark.parametrize("t", [Q4_0, Q8_0, IQ4_NL])
@pytest.mark.parametrize("M,K,N", [
    (10, 256, 4),        # one stretch, three of four row tiles empty
    (16, 768, 132),      # K = one slice and a half, weight rows not a multiple of 32
    (33, 1280, 256),     # two column tiles
    (64, 2304, 300),     # K not a multiple of the slice length
    (12, 96, 64),        # K not a multiple of 256: not this kernel's
    (24, 8192, 20000),   # enough work for the longest slices
    (40, 4096, 4096),
    (96, 512, 512),      # three column tiles
    (8, 1024, 36),
])
def test_split_k_small_batches_q8_q4(gpu, oracle, t, M, K, N):
    """8 .. 96 rows (the range extends to 192 by shape) of Q8_0 / Q4_0 / IQ4_NL (N a multiple of 4, K of 256): the split-K MFMA kernel
    with exact integer weight operands; x -> fp16 is its only rounding."""
    W = synth.weights(t, 70 + t, N, K)
    x = synth.activations(71 + t, M, K)
    bias = synth.normal(72 + t, 0, N).astype(np.float32) * 0.1
    for act in (0, 1):
        got = run_dense(gpu, t, x, W, bias, act)
        want = oracle.c_qdense(t, x, W, bias, act)
        assert rel_err(got, want) < TOL_F32, (t, M, K, N, act)
    # bf16 activations widen exactly into the kernel's fp16 image: same bound (the shape that is not
    # this kernel's takes a bf16 MFMA path)
    xb = bf16_round(x)
    tol = TOL_F32 if K % 256 == 0 else TOL_BF16
    assert rel_err(run_dense(gpu, t, xb, W, bias, 0, bf16=True), oracle.c_qdense(t, xb, W, bias, 0)) < tol, (t, M, K, N, "bf16")


@pytest.mark.parametrize("t,M,K,N", [(Q8_0, 192, 1024, 256), (Q4_0, 160, 2048, 132), (Q4_0, 97, 4096, 64), (Q4_K, 128, 1024, 260),
                                     (Q4_K, 100, 2048, 36), (Q6_K, 96, 1024, 64), (Q6_K, 70, 2560, 128), (IQ4_NL, 192, 512, 128)])
def test_split_k_up_to_six_tiles_of_batch_rows(gpu, oracle, t, M, K, N):
    """Where the two-pass GEMM is the dearer route (small and long-K matrices) the split-K kernels serve up to 192 rows:
    several tiles of 32 batch rows, the last one partly filled."""
    W = synth.weights(t, 170 + t, N, K)
    x = (synth.activations(171 + t, M, K) * np.logspace(-3, 3, M, dtype=np.float32)[:, None]).astype(np.float32)
    bias = synth.normal(172 + t, 0, N).astype(np.float32) * 0.1
    got = run_dense(gpu, t, x, W, bias, 0)
    want = oracle.c_qdense(t, x, W, bias, 0)
    per_row = np.max(np.abs(got.astype(np.float64) - want), axis=1) / np.max(np.abs(want), axis=1)
    assert np.all(per_row < TOL_F32), (t, M, K, N, float(per_row.max()))


@pytest.mark.parametrize("t", [Q4_K, Q6_K])
@pytest.mark.parametrize("M,K,N", [(8, 512, 8), (32, 2048, 260), (70, 4096, 512), (96, 1024, 4096), (33, 1536, 100), (12, 7680, 36)])
def test_split_k_small_batches_k_quants(gpu, oracle, t, M, K, N):
    """Small batches of Q4_K and Q6_K, fp32 and bf16 activations, through the split-K MFMA kernels
    (K a multiple of 512; 1536 and 7680 leave the last 1024-value slice of Q6_K half empty)."""
    W = synth.weights(t, 75, N, K)
    x = synth.activations(76, M, K)
    bias = synth.normal(77, 0, N).astype(np.float32) * 0.1
    assert rel_err(run_dense(gpu, t, x, W, bias, 3), oracle.c_qdense(t, x, W, bias, 3)) < TOL_F32, (t, M, K, N, "f32")
    xb = bf16_round(x)
    tol = TOL_F32 if (t == Q4_K or M <= 32) else TOL_BF16  # Q6_K beyond 32 rows takes the bf16 MFMA GEMM on these matrices
    assert rel_err(run_dense(gpu, t, xb, W, bias, 3, bf16=True), oracle.c_qdense(t, xb, W, bias, 3)) < tol, (t, M, K, N, "bf16")


def test_q4_k_split_k_walks_several_batch_tiles_together(gpu, oracle):
    """More than 32 batch rows on the Q4_K split-K route: one launch contracts up to four tiles of 32 rows against every weight
    tile (codes converted once).  A long-K matrix of 25.6 MB, which keeps the route up to 320 rows: every tile count, further
    launches for the rows past 128 (tiles dealt evenly: 3 + 2, 4 + 4, 4 + 3 + 3), a last tile that is partly filled, a width that is not a multiple of the workgroup's 256
    rows; fp32 and bf16 activations; the gated pair, the projection with normalisation and residual, and q / k / v."""
    t, K, N = Q4_K, 14336, 3172
    assert N * ggml.row_bytes(t, K) >= 24 << 20
    q = Quantization(ggml_type=t)
    W = synth.weights(t, 1500, N, K)
    bias = synth.normal(1501, 0, N).astype(np.float32) * 0.1
    Wd = dev(gpu, W)
    x_all = synth.activations(1502, 320, K)
    want_all = oracle.c_qdense(t, x_all, W, bias, 3)  # (rows are independent: one oracle pass serves every batch size)
    for M in (33, 64, 70, 96, 128, 129, 160, 250, 320):
        got = nn.quantized_dense(dev(gpu, np.ascontiguousarray(x_all[320 - M:])), Wd, q, dev(gpu, bias), BACKEND_ACT[3]).cpu().numpy()
        assert rel_err(got, want_all[320 - M:]) < TOL_F32, M
    xb = bf16_round(synth.activations(1510, 100, K))
    assert rel_err(run_dense(gpu, t, xb, W, bias, 0, bf16=True), oracle.c_qdense(t, xb, W, bias, 0)) < TOL_F32
    # projection with normalisation and residual
    M = 100
    gain = (synth.normal(1511, 0, K) * 0.5 + 1.0).astype(np.float32)
    cfg = nn.RMSNorm(dev(gpu, gain), 1e-6, 0.0)
    x = (synth.activations(1512, M, K) * 2.0).astype(np.float32)
    xn = oracle.c_rmsnorm(x, gain, 1e-6, 0.0)
    res = synth.activations(1513, M, N)
    got = nn.quantized_dense(dev(gpu, x), Wd, q, None, BACKEND_ACT[0], norm=cfg, residual=dev(gpu, res)).cpu().numpy()
    dense = oracle.c_qdense(t, xn, W)
    assert float(np.max(np.abs(got.astype(np.float64) - (dense + res)))) / float(np.max(np.abs(dense))) < TOL_F32
    # q / k / v of one normalised input: 2048 + 512 + 612 rows side by side
    parts = [(0, 2048), (2048, 2560), (2560, 3172)]
    outs = nn.quantized_dense_batch([(dev(gpu, x), dev(gpu, np.ascontiguousarray(W[a:b])), q, None, None) for a, b in parts], norm=cfg)
    gpu.cuda.synchronize()
    for (a, b), y in zip(parts, outs):
        assert rel_err(y.cpu().numpy(), dense[:, a:b]) < TOL_F32, (a, b)
    # gated pair
    assert gated_case(gpu, oracle, t, 96, K, 1028, 3, 1, True, 1520) < 2 * TOL_F32
    assert gated_case(gpu, oracle, t, 130, 4096, 2052, 3, 0, False, 1530) < 2 * TOL_F32
    assert gated_case(gpu, oracle, t, 170, 4096, 11008, 3, 1, True, 1540) < 2 * TOL_F32  # (a wide pair of 25 MB each keeps the route past 160 rows, up to 384)


@pytest.mark.parametrize("t", [Q4_0, IQ4_NL, Q8_0])
def test_32_value_block_formats_walk_several_batch_tiles_together(gpu, oracle, t):
    """Q4_0, IQ4_NL and Q8_0 at more than 32 batch rows on the split-K route (up to 128 rows and more): one launch contracts two
    to four tiles of 32 rows against every parked stretch of weights (Q8_0: one parked stretch, the next one through registers).  A width that is not a multiple of the workgroup's 256 rows, a last
    tile that is partly filled, slices of 512 and of 1024 values with a shorter last one, a long-K matrix; fp32 and bf16
    activations, a projection with normalisation and residual, a gated pair."""
    q = Quantization(ggml_type=t)
    # (the kernel serves matrices whose 256-row workgroups times 512-value slices cover three quarters of the CUs)
    for K, N in ((4096, 6148), (4096 + 768, 5124), (14336, 1796)):
        W = synth.weights(t, 1600 + t, N, K)
        bias = synth.normal(1601, 0, N).astype(np.float32) * 0.1
        x_all = synth.activations(1602 + K, 128, K)
        want_all = oracle.c_qdense(t, x_all, W, bias, 3)  # (rows are independent: one oracle pass serves every batch size)
        for M in (33, 64, 70, 97, 128):
            got = nn.quantized_dense(dev(gpu, np.ascontiguousarray(x_all[128 - M:])), dev(gpu, W), q, dev(gpu, bias), BACKEND_ACT[3]).cpu().numpy()
            assert rel_err(got, want_all[128 - M:]) < TOL_F32, (ggml.name(t), K, N, M)
        xb = bf16_round(x_all[:100])
        assert rel_err(run_dense(gpu, t, xb, W, bias, 0, bf16=True), oracle.c_qdense(t, xb, W, bias, 0)) < TOL_F32, (ggml.name(t), K, N, "bf16")
    K, N, M = 4096, 6148, 100
    W = synth.weights(t, 1610 + t, N, K)
    gain = (synth.normal(1611, 0, K) * 0.5 + 1.0).astype(np.float32)
    x = (synth.activations(1612, M, K) * 2.0).astype(np.float32)
    res = synth.activations(1613, M, N)
    got = nn.quantized_dense(dev(gpu, x), dev(gpu, W), q, None, BACKEND_ACT[0], norm=nn.RMSNorm(dev(gpu, gain), 1e-6, 0.0),
                             residual=dev(gpu, res)).cpu().numpy()
    dense = oracle.c_qdense(t, oracle.c_rmsnorm(x, gain, 1e-6, 0.0), W)
    assert float(np.max(np.abs(got.astype(np.float64) - (dense + res)))) / float(np.max(np.abs(dense))) < TOL_F32, ggml.name(t)
    assert gated_case(gpu, oracle, t, 100, 4096, 3076, 3, 1, True, 1620) < 2 * TOL_F32
    assert gated_case(gpu, oracle, t, 70, 2048, 516, 3, 0, False, 1630) < 2 * TOL_F32  # (a small pair: one launch per 32 rows)


def test_q4_k_large_minima_through_the_split_k_kernel(gpu, oracle):
    """Q4_K super-blocks whose minimum term is as large as the format allows to matter: dmin = 2048 with every 6-bit minimum at
    63 (dmin * m = 129 024 lies beyond the largest fp16, 65 504, and has 17 significant bits).  The small-batch kernel must
    carry dmin in fp32, as the decode GEMV and the dequantisation do: 8 and 32 rows against the oracle, and against the
    one-row result of the same activations."""
    N, K = 256, 2048
    W = synth.weights(Q4_K, 91, N, K).copy().reshape(N, K // 256, 144)
    W[:, :, 2:4] = np.frombuffer(np.float16(2048.0).tobytes(), dtype=np.uint8)   # dmin
    W[:, :, 0:2] = np.frombuffer(np.float16(0.5).tobytes(), dtype=np.uint8)      # d
    sc = W[:, :, 4:16].copy()                   # the 12 bytes of packed 6-bit scales and minima
    sc[:, :, 4:8] = 0xFF                        # m0..m3 = 63 (low six bits) and the two high bits of m4..m7
    sc[:, :, 8:12] |= 0xF0                      # the low four bits of m4..m7
    W[:, :, 4:16] = sc
    W = W.reshape(N, -1)
    for M in (8, 32):
        x = synth.activations(92, M, K)
        want = oracle.c_qdense(Q4_K, x, W, None, 0)
        got = run_dense(gpu, Q4_K, x, W)
        assert np.all(np.isfinite(got)), M
        assert rel_err(got, want) < TOL_F32, (M, rel_err(got, want))
        one = np.concatenate([run_dense(gpu, Q4_K, x[m:m + 1], W) for m in range(2)])
        assert rel_err(got[:2], one) < TOL_F32, M


@pytest.mark.parametrize("t", [Q6_K, Q4_K])
def test_output_head_of_a_128k_vocabulary(gpu, oracle, t):
    """The largest projection of a decoder: hidden state -> logits over 128 256 tokens (K = 4096; several hundred
    megabytes of weights, row offsets beyond 2^28 bytes).  One row and a small batch, checked on a sample of 3000
    output columns that includes the first and the last."""
    K, N = 4096, 128256
    W = synth.weights(t, 480 + t, N, K)
    rng = np.random.default_rng(481)
    cols = np.unique(np.concatenate([[0, 1, N - 2, N - 1], rng.integers(0, N, 3000)]))
    for M in (1, 8, 40):
        x = synth.activations(482 + M, M, K)
        got = run_dense(gpu, t, x, W)
        assert got.shape == (M, N) and np.all(np.isfinite(got))
        want = oracle.c_qdense(t, x, np.ascontiguousarray(W[cols]))
        assert rel_err(got[:, cols], want) < TOL_F32, (t, M)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_gemv_long_k_is_chunked(gpu, oracle, t):
    """K above the 16384 values one LDS pass holds."""
    K, N = 16384 + 4096, 19
    W = synth.weights(t, 30 + t, N, K)
    x = synth.activations(31 + t, 1, K)
    assert rel_err(run_dense(gpu, t, x, W), oracle.c_qdense(t, x, W)) < TOL_F32


@pytest.mark.parametrize("t", ALL_TYPES)
def test_gemv_all_activations_and_no_bias(gpu, oracle, t):
    K, N = 512, 96
    W = synth.weights(t, 40 + t, N, K)
    x = synth.activations(41 + t, 1, K)
    # scale so pre-activations spread over roughly [-4, 4]
    pre = oracle.c_qdense(t, x, W)
    x = (x * (2.0 / (np.std(pre) + 1e-9))).astype(np.float32)
    for act in range(6):
        got = run_dense(gpu, t, x, W, None, act)
        want = oracle.c_qdense(t, x, W, None, act)
        assert rel_err(got, want) < TOL_F32, (t, act)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_gemv_unit_vectors_return_dequantised_columns(gpu, oracle, t):
    K, N = 512, 40
    W = synth.weights(t, 50 + t, N, K)
    Wd = oracle.c_dequantize(t, W, K)
    for k in [0, 15, 16, 31, 32, 63, 255, 256, 300, 511]:
        x = np.zeros((1, K), np.float32)
        x[0, k] = 1.0
        got = run_dense(gpu, t, x, W)[0]
        # Q4_K values are a difference (d*sc*q - dmin*m): allow the rounding of the larger terms
        np.testing.assert_allclose(got, Wd[:, k], rtol=2e-6, atol=1e-6 * float(np.max(np.abs(Wd[:, k]))))


def test_gemv_unaligned_activation_pointer(gpu, oracle):
    K, N = 1024, 50
    W = synth.weights(Q4_0, 60, N, K)
    x = synth.activations(61, 1, K)
    buf = gpu.zeros(K + 1, dtype=gpu.float32, device="cuda")
    buf[1:] = dev(gpu, x[0])
    xv = buf[1:].view(1, K)  # 4-byte aligned only
    y = nn.quantized_dense(xv, dev(gpu, W), Quantization(ggml_type=Q4_0))
    assert rel_err(y.cpu().numpy(), oracle.c_qdense(Q4_0, x, W)) < TOL_F32


@pytest.mark.parametrize("t", [Q4_0, Q8_0, IQ4_NL])
@pytest.mark.parametrize("K", [32, 96, 160])
def test_batched_ragged_k_steps(gpu, oracle, t, K):
    """K that is not a multiple of the kernels' K step (32-value blocks only)."""
    M, N = 9, 21
    W = synth.weights(t, 300 + K, N, K)
    x = synth.activations(301 + K, M, K)
    assert rel_err(run_dense(gpu, t, x, W), oracle.c_qdense(t, x, W)) < TOL_F32
    xb = bf16_round(x)
    assert rel_err(run_dense(gpu, t, xb, W, bf16=True), oracle.c_qdense(t, xb, W)) < TOL_BF16
    x1 = x[:1]
    assert rel_err(run_dense(gpu, t, x1, W), oracle.c_qdense(t, x1, W)) < TOL_F32


def test_leading_batch_axes_and_empty_batch(gpu, oracle):
    K, N = 256, 12
    W = synth.weights(Q8_0, 70, N, K)
    x = synth.activations(71, 6, K).reshape(2, 3, K)
    y = nn.quantized_dense(dev(gpu, x), dev(gpu, W), Quantization(ggml_type=Q8_0))
    assert tuple(y.shape) == (2, 3, N)
    assert rel_err(y.cpu().numpy().reshape(6, N), oracle.c_qdense(Q8_0, x.reshape(6, K), W)) < TOL_F32
    y0 = nn.quantized_dense(gpu.zeros((0, K), device="cuda"), dev(gpu, W), Quantization(ggml_type=Q8_0))
    assert tuple(y0.shape) == (0, N)


# ------------------------------------------------------------------------------ batched (MFMA) paths

@pytest.mark.parametrize("t", ALL_TYPES)
@pytest.mark.parametrize("M,K,N", [(5, 256, 7), (32, 1024, 130), (130, 512, 257), (64, 4096, 96), (300, 768, 40)])
def test_batched_f32_parity(gpu, oracle, t, M, K, N):
    W = synth.weights(t, 80 + t, N, K)
    x = synth.activations(81 + t, M, K)
    bias = synth.normal(82 + t, 0, N).astype(np.float32) * 0.1
    for act in (0, 2):
        got = run_dense(gpu, t, x, W, bias, act)
        want = oracle.c_qdense(t, x, W, bias, act)
        assert rel_err(got, want) < TOL_F32, (t, M, K, N, act)


@pytest.mark.parametrize("t", ALL_TYPES)
@pytest.mark.parametrize("M,K,N", [(1, 256, 5), (64, 1024, 130), (200, 512, 300), (260, 768, 129)])
def test_bf16_prefill_parity(gpu, oracle, t, M, K, N):
    W = synth.weights(t, 90 + t, N, K)
    x = bf16_round(synth.activations(91 + t, M, K))
    bias = synth.normal(92 + t, 0, N).astype(np.float32) * 0.1
    got = run_dense(gpu, t, x, W, bias, 3, bf16=True)
    want = oracle.c_qdense(t, x, W, bias, 3)
    assert rel_err(got, want) < TOL_BF16, (t, M, K, N)


@pytest.mark.parametrize("t", ALL_TYPES)
@pytest.mark.parametrize("M,K,N", [
    (512, 256, 130),    # smallest batch of the two-pass path; four K steps; ragged last weight tile
    (513, 512, 128),    # one row into a third activation tile
    (700, 768, 300),    # twelve K steps: the stage ring wraps four times
    (1024, 1280, 64),   # twenty steps, half a weight tile
])
def test_large_batches_two_pass(gpu, oracle, t, M, K, N):
    """Batches of 512 rows and more dequantise W once into a 16-bit image and run a plain MFMA
    GEMM whose operands go from global memory straight into LDS."""
    W = synth.weights(t, 95 + t, N, K)
    bias = synth.normal(96 + t, 0, N).astype(np.float32) * 0.1
    x = synth.activations(97 + t, M, K)
    want = oracle.c_qdense(t, x, W, bias, 2)
    assert rel_err(run_dense(gpu, t, x, W, bias, 2), want) < TOL_F32, (t, M, K, N, "f32")
    xb = bf16_round(x)
    want = oracle.c_qdense(t, xb, W, None, 0)
    assert rel_err(run_dense(gpu, t, xb, W, None, 0, bf16=True), want) < TOL_BF16, (t, M, K, N, "bf16")


@pytest.mark.parametrize("t", [Q4_0, Q8_0, IQ4_NL])
@pytest.mark.parametrize("M,K,N", [
    (17, 64, 40),       # one K step, less than one weight tile
    (33, 128, 64),      # two K steps, exactly one 64-row weight tile
    (64, 192, 130),     # three K steps, ragged last weight tile
    (100, 1024, 300),   # sixteen K steps
    (128, 4096, 257),   # a full tile of activation rows
    (20, 256, 40000),   # enough weight tiles for the largest tile
])
def test_batches_of_17_to_128_rows(gpu, oracle, t, M, K, N):
    """The batch sizes between the GEMV passes and a full tile of activation rows, where the small
    tiles of the 16-bit GEMM are chosen; few K steps, ragged weight tiles, both activation types."""
    W = synth.weights(t, 85 + t, N, K)
    bias = synth.normal(86 + t, 0, N).astype(np.float32) * 0.1
    x = synth.activations(87 + t, M, K)
    want = oracle.c_qdense(t, x, W, bias, 3)
    assert rel_err(run_dense(gpu, t, x, W, bias, 3), want) < TOL_F32, (t, M, K, N, "f32")
    xb = bf16_round(x)
    want = oracle.c_qdense(t, xb, W, None, 0)
    assert rel_err(run_dense(gpu, t, xb, W, None, 0, bf16=True), want) < TOL_BF16, (t, M, K, N, "bf16")


@pytest.mark.parametrize("K", [64, 128, 192, 96])
def test_large_batches_few_k_steps(gpu, oracle, K):
    """One, two and three K steps (shorter than the stage ring) and a K that is not a multiple of
    64, which for bf16 activations (read in place) stays on the fused kernel."""
    M, N = 600, 200
    W = synth.weights(Q8_0, 98, N, K)
    x = bf16_round(synth.activations(99, M, K))
    want = oracle.c_qdense(Q8_0, x, W, None, 0)
    assert rel_err(run_dense(gpu, Q8_0, x, W, None, 0, bf16=True), want) < TOL_BF16, K


def _boundary_cases():
    """Seeded random problems around every batch-size threshold of the dispatcher."""
    rng = np.random.default_rng(20240607)
    rows = [1, 2, 4, 5, 7, 8, 9, 16, 17, 31, 32, 33, 64, 95, 96, 97, 128, 129, 256, 257, 300, 511, 512, 513]
    cases = []
    for i, M in enumerate(rows):
        for rep in range(2):
            t = ALL_TYPES[(i + 2 * rep) % len(ALL_TYPES)]
            big = t in (Q4_K, Q6_K)
            if rep == 0:
                K = int(rng.choice([256, 512, 768, 1024, 2048]))
            else:
                K = int(rng.choice([256, 1280]) if big else rng.choice([32, 96, 160, 544, 1056]))
            N = int(rng.choice([4, 36, 64, 100, 132, 257, 512, 600]))
            cases.append((t, M, K, N, bool((i + rep) % 2), int(rng.integers(0, 6)), bool(rng.integers(0, 2))))
    return cases


@pytest.mark.parametrize("t,M,K,N,bf16,act,with_bias", _boundary_cases())
def test_dispatch_boundaries(gpu, oracle, t, M, K, N, bf16, act, with_bias):
    """The error is measured against the larger of the output and the pre-activation magnitude: a
    saturating activation (tanh) shrinks the outputs but not the error of the contraction that
    feeds it (all six activations have slope <= 1.13), and the bound is on that contraction."""
    W = synth.weights(t, 300 + M, N, K)
    x = synth.activations(301 + M, M, K)
    bias = synth.normal(302 + M, 0, N).astype(np.float32) * 0.1 if with_bias else None
    if bf16:
        x = bf16_round(x)
    got = run_dense(gpu, t, x, W, bias, act, bf16=bf16)
    want = oracle.c_qdense(t, x, W, bias, act)
    pre = oracle.c_qdense(t, x, W, bias, 0)
    assert got.shape == (M, N)
    scale = max(float(np.max(np.abs(want))), float(np.max(np.abs(pre)))) or 1.0
    err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) / scale
    assert err < (TOL_BF16 if bf16 else TOL_F32), (t, M, K, N, bf16, act, err)


@pytest.mark.parametrize("t,N", [(Q8_0, 6400), (Q4_0, 11264), (Q4_K, 11264), (Q6_K, 8192), (IQ4_NL, 11264)])
def test_small_batches_on_large_matrices(gpu, oracle, t, N):
    """Matrices of 24 MB and more: batches of 2 .. 8 rows run as GEMV passes of up to four rows against one
    reading of W (remainders of 1, 2, 3 rows included) and hand over to the split-K kernels after 5 - 7 rows."""
    K = 4096
    assert N * ggml.row_bytes(t, K) >= 24 << 20
    W = synth.weights(t, 330 + t, N, K)
    bias = synth.normal(331 + t, 0, N).astype(np.float32) * 0.1
    for M in (2, 3, 4, 5, 6, 7, 8):
        x = synth.activations(332 + M, M, K)
        want = oracle.c_qdense(t, x, W, bias, 3)
        assert rel_err(run_dense(gpu, t, x, W, bias, 3), want) < TOL_F32, (t, M)
    for M in (3, 5):
        xb = bf16_round(synth.activations(340 + M, M, K))
        assert rel_err(run_dense(gpu, t, xb, W, bias, 3, bf16=True), oracle.c_qdense(t, xb, W, bias, 3)) < TOL_BF16, (t, M)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_hand_over_from_split_k_to_the_two_passes(gpu, oracle, t):
    """A 4096 x 2048 matrix (between 6 and 24 MB in every format): the split-K kernels hand over to the two-pass GEMM after
    64, 96 or 128 rows depending on the format; both sides of each of those points and of 160, fp32 and bf16 activations."""
    K, N = 4096, 2048 if t != Q4_0 and t != IQ4_NL and t != Q4_K else 3072
    assert 6 << 20 <= N * ggml.row_bytes(t, K) < 24 << 20
    W = synth.weights(t, 350 + t, N, K)
    for M in (64, 65, 96, 97, 128, 129, 160, 161):
        x = synth.activations(351 + M, M, K)
        assert rel_err(run_dense(gpu, t, x, W), oracle.c_qdense(t, x, W)) < TOL_F32, (t, M)
    for M in (65, 97, 129):
        xb = bf16_round(synth.activations(360 + M, M, K))
        assert rel_err(run_dense(gpu, t, xb, W, bf16=True), oracle.c_qdense(t, xb, W)) < TOL_BF16, (t, M)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_few_rows_on_few_columns_split_k_inside_the_gemm(gpu, oracle, t):
    """Past the split-K kernels' range a narrow matrix gives the GEMM fewer tiles than the chip has CUs; K is then cut into up
    to eight slices whose sums a small kernel adds up and finishes (row scales, bias, activation, residual).  Dense calls
    with fp32 and bf16 activations, a projection with normalisation and residual, q / k / v behind one normalisation;
    slices of equal and unequal length; a width that is not a multiple of 4 keeps the unsplit GEMM."""
    q = Quantization(ggml_type=t)
    for M, K, N, act in ((200, 4096, 512, 3), (130, 2304, 1024, 0), (300, 3328, 256, 2), (200, 4096, 510, 1), (17, 8192, 64, 0), (130, 14336, 256, 0)):
        W = synth.weights(t, 1400 + t, N, K)
        bias = synth.normal(1401, 0, N).astype(np.float32) * 0.1
        x = synth.activations(1402 + M, M, K)
        assert rel_err(run_dense(gpu, t, x, W, bias, act), oracle.c_qdense(t, x, W, bias, act)) < TOL_F32, (ggml.name(t), M, K, N)
        xb = bf16_round(x)
        assert rel_err(run_dense(gpu, t, xb, W, None, act, bf16=True), oracle.c_qdense(t, xb, W, None, act)) < TOL_BF16, (ggml.name(t), M, K, N)
    for M, K, N in ((130, 10240, 256), (200, 4096, 512)):  # (rows of more than 8192 values: 64 per thread in the activation pass)
        W = synth.weights(t, 1410 + t, N, K)
        gain = (synth.normal(1411, 0, K) * 0.5 + 1.0).astype(np.float32)
        cfg = nn.RMSNorm(dev(gpu, gain), 1e-6, 0.0)
        x = (synth.activations(1412, M, K) * 2.0).astype(np.float32)
        xn = oracle.c_rmsnorm(x, gain, 1e-6, 0.0)
        res = synth.activations(1413, M, N)
        got = nn.quantized_dense(dev(gpu, x), dev(gpu, W), q, None, BACKEND_ACT[0], norm=cfg, residual=dev(gpu, res)).cpu().numpy()
        dense = oracle.c_qdense(t, xn, W)
        assert float(np.max(np.abs(got.astype(np.float64) - (dense + res)))) / float(np.max(np.abs(dense))) < TOL_F32, (ggml.name(t), K)
    Ws = [synth.weights(t, 1420 + j, n, K) for j, n in enumerate((512, 128, 128))]
    bs = [synth.normal(1425, 0, 512).astype(np.float32) * 0.1, None, None]
    outs = nn.quantized_dense_batch([(dev(gpu, x), dev(gpu, Wj), q, None if b is None else dev(gpu, b), None) for Wj, b in zip(Ws, bs)], norm=cfg)
    gpu.cuda.synchronize()
    for Wj, b, y in zip(Ws, bs, outs):
        assert rel_err(y.cpu().numpy(), oracle.c_qdense(t, xn, Wj, b)) < TOL_F32, (ggml.name(t), Wj.shape)


@pytest.mark.parametrize("t,N", [(Q8_0, 3328), (Q4_K, 5632), (Q6_K, 4096)])
def test_small_batches_with_neighbours_on_large_matrices(gpu, oracle, t, N):
    """The same batches through the calls around a projection: passes of two rows inside the decode GEMV up to the
    measured change-over of each format and matrix class (3 to 8 rows), the split-K kernels with the extras beyond."""
    K = 4096
    assert 2 * N * ggml.row_bytes(t, K) >= 24 << 20
    for i, M in enumerate((2, 3, 4, 5, 7, 8)):
        err = gated_case(gpu, oracle, t, M, K, N, 3, 1 + i % 3, bool(i % 2), 350 + 10 * i + t)
        assert err < 2 * TOL_F32, ("gated", t, M, err)
    N2 = 2 * N
    W = synth.weights(t, 360 + t, N2, K)
    gain = (synth.normal(361, 0, K) * 0.5 + 1.0).astype(np.float32)
    for M in (2, 3, 4, 5, 6):
        x = (synth.activations(362 + M, M, K) * 2.0).astype(np.float32)
        res = synth.activations(363 + M, M, N2)
        got = nn.quantized_dense(dev(gpu, x), dev(gpu, W), Quantization(ggml_type=t), None, BACKEND_ACT[0],
                                 norm=nn.RMSNorm(dev(gpu, gain), 1e-6, 0.0), residual=dev(gpu, res)).cpu().numpy()
        dense = oracle.c_qdense(t, oracle.c_rmsnorm(x, gain, 1e-6, 0.0), W)
        err = float(np.max(np.abs(got.astype(np.float64) - (dense + res)))) / float(np.max(np.abs(dense)))
        assert err < TOL_F32, ("block", t, M, err)


@pytest.mark.parametrize("t", [Q4_0, Q8_0, IQ4_NL])
def test_small_batches_over_a_single_block_are_exact_passes(gpu, oracle, t):
    """K of one or a few blocks leaves no averaging for 16-bit operands to lean on: batches of 5 .. 16 rows
    on such shapes run as fp32 passes and stay well inside the bound (a seeded sweep once found 1.25e-3
    on a 7 x 32 x 8 problem through the fp16-operand GEMM)."""
    for M, K, N in ((7, 32, 8), (16, 96, 5), (5, 160, 33), (12, 544, 16)):
        W = synth.weights(t, 380 + M, N, K)
        x = synth.activations(381 + M, M, K)
        bias = synth.normal(382 + M, 0, N).astype(np.float32) * 0.1
        for seed in range(3):
            x = synth.activations(383 + 7 * seed + M, M, K)
            assert rel_err(run_dense(gpu, t, x, W, bias, 0), oracle.c_qdense(t, x, W, bias, 0)) < 1e-4, (t, M, K, N)


@pytest.mark.parametrize("t", [Q8_0, Q4_K, Q6_K])
def test_activation_magnitude_does_not_matter(gpu, oracle, t):
    """The reference computes in fp32 and is indifferent to the scale of x.  So is every kernel family
    here: the GEMV quantises every 32 activations on their own, the MFMA paths scale every batch row
    (split-K: every K-slice of it) by a power of two before rounding to fp16.  Rows of very different
    magnitude in one batch included."""
    K, N = 1024, 256
    W = synth.weights(t, 390 + t, N, K)
    for M in (1, 3, 8, 32, 300):
        base = synth.activations(391 + M, M, K)
        for sc in (1e-7, 1e-4, 1.0, 3e4, 1e9):
            x = (base * np.float32(sc)).astype(np.float32)
            got = run_dense(gpu, t, x, W)
            assert rel_err(got, oracle.c_qdense(t, x, W)) < TOL_F32, (t, M, sc)
        if M > 1:
            rows = (base * np.logspace(-6, 8, M, dtype=np.float32)[:, None]).astype(np.float32)
            got = run_dense(gpu, t, rows, W)
            want = oracle.c_qdense(t, rows, W)
            per_row = np.max(np.abs(got.astype(np.float64) - want), axis=1) / np.max(np.abs(want), axis=1)
            assert np.all(per_row < TOL_F32), (t, M, float(per_row.max()))


@pytest.mark.parametrize("t", [Q8_0, Q4_0, IQ4_NL])
def test_large_batches_over_an_odd_number_of_blocks(gpu, oracle, t):
    """K an odd multiple of 32 with more than 16 fp32 rows: both 16-bit images get rows padded with
    zeros to the GEMM's step of 64, so these shapes take the two scaled passes like every other and
    are as indifferent to the magnitude of x; with the neighbours of a decoder block as well."""
    for i, (M, K, N) in enumerate([(17, 32, 8), (40, 96, 130), (300, 160, 257), (130, 1056, 132)]):
        W = synth.weights(t, 440 + i, N, K)
        base = synth.activations(441 + i, M, K)
        bias = synth.normal(442 + i, 0, N).astype(np.float32) * 0.1
        for sc in (1e-7, 1.0, 1e9):
            x = (base * np.float32(sc)).astype(np.float32)
            assert rel_err(run_dense(gpu, t, x, W), oracle.c_qdense(t, x, W)) < TOL_F32, (t, M, K, N, sc)
        got = run_dense(gpu, t, base, W, bias, 3)
        want, pre = oracle.c_qdense(t, base, W, bias, 3), oracle.c_qdense(t, base, W, bias, 0)
        err = float(np.max(np.abs(got.astype(np.float64) - want))) / max(float(np.max(np.abs(want))), float(np.max(np.abs(pre))))
        assert err < TOL_F32, (t, M, K, N, err)
        for norm_kind in (0, 1):
            err = gated_case(gpu, oracle, t, M, K, N, 3, norm_kind, True, 450 + 10 * i + t)
            assert err < 2 * TOL_F32, ("gated", t, M, K, N, norm_kind, err)


def test_randomized_problems(gpu, oracle):
    """150 seeded random problems over all formats, both activation types, every activation, with
    and without bias: batch sizes, K and N drawn from lists that include every tile and slice
    boundary of the kernels.  Error measured on the contraction scale as above."""
    rng = np.random.default_rng(7)
    rows = [1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17, 24, 32, 33, 48, 64, 65, 96, 97, 100, 128, 130, 200, 256, 257, 300, 512, 700, 1024]
    done = 0
    while done < 150:
        t = ALL_TYPES[int(rng.integers(0, len(ALL_TYPES)))]
        big = t in (Q4_K, Q6_K)
        M = int(rng.choice(rows))
        K = (256 if big else 32) * int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17, 20] if big else
                                                 [1, 2, 3, 5, 8, 9, 16, 17, 24, 32, 33, 48, 64, 96, 128, 136]))
        N = int(rng.choice([1, 3, 4, 8, 31, 32, 33, 64, 100, 128, 129, 200, 256, 300, 512, 777, 1024]))
        bf16, act, with_bias = bool(rng.integers(0, 2)), int(rng.integers(0, 6)), bool(rng.integers(0, 2))
        if M * K * N > 3e8:
            continue
        done += 1
        W = synth.weights(t, 5000 + done, N, K)
        x = synth.activations(6000 + done, M, K)
        bias = synth.normal(7000 + done, 0, N).astype(np.float32) * 0.1 if with_bias else None
        if bf16:
            x = bf16_round(x)
        got = run_dense(gpu, t, x, W, bias, act, bf16=bf16)
        want = oracle.c_qdense(t, x, W, bias, act)
        pre = oracle.c_qdense(t, x, W, bias, 0)
        scale = max(float(np.max(np.abs(want))), float(np.max(np.abs(pre)))) or 1.0
        err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) / scale
        assert np.all(np.isfinite(got)) and err < (TOL_BF16 if bf16 else TOL_F32), (t, M, K, N, bf16, act, with_bias, err)


# ------------------------------------------------------------------------------ callers around the dense layers

def test_rmsnorm_reference_kat(gpu, kats):
    for k in kats["rmsnorm"]:
        x = np.array(k["x"], np.float32)
        got = nn.rms_norm(dev(gpu, x), nn.RMSNorm(epsilon=k["eps"])).cpu().numpy()
        np.testing.assert_allclose(got, np.array(k["want"], np.float32), rtol=0, atol=k["tol"], err_msg=k["name"])
        ones = dev(gpu, np.ones(x.shape[-1], np.float32))
        got = nn.rms_norm(dev(gpu, x), nn.RMSNorm(gain=ones, epsilon=k["eps"])).cpu().numpy()
        np.testing.assert_allclose(got, np.array(k["want"], np.float32), rtol=0, atol=k["tol"], err_msg=k["name"])


@pytest.mark.parametrize("M,K", [(1, 1), (3, 33), (2, 4096), (70, 1000)])
def test_rmsnorm_parity(gpu, oracle, M, K):
    x = (synth.activations(300, M, K) * 2.5).astype(np.float32)
    gain = synth.normal(301, 0, K).astype(np.float32)
    for g, eps, off in ((None, 1e-6, 0.0), (gain, 1e-5, 0.0), (gain, 1e-6, 1.0), (None, 0.0, 0.0)):
        got = nn.rms_norm(dev(gpu, x), nn.RMSNorm(None if g is None else dev(gpu, g), eps, off)).cpu().numpy()
        want = oracle.c_rmsnorm(x, g, eps, off)
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-30)


def gated_case(gpu, oracle, t, M, K, N, act, norm_kind, with_bias, seed):
    Wg, Wu = synth.weights(t, seed, N, K), synth.weights(t, seed + 1, N, K)
    x = synth.activations(seed + 2, M, K)
    gain = (synth.normal(seed + 3, 0, K) * 0.5 + 1.0).astype(np.float32)
    bg = synth.normal(seed + 4, 0, N).astype(np.float32) * 0.1 if with_bias else None
    bu = synth.normal(seed + 5, 0, N).astype(np.float32) * 0.1 if with_bias else None
    norm = {0: None, 1: (gain, 1e-6, 0.0), 2: (gain, 1e-5, 1.0), 3: (None, 1e-6, 0.0)}[norm_kind]
    cfg = None if norm is None else nn.RMSNorm(None if norm[0] is None else dev(gpu, norm[0]), norm[1], norm[2])
    got = nn.gated_feed_forward(dev(gpu, x), dev(gpu, Wg), dev(gpu, Wu), Quantization(ggml_type=t), BACKEND_ACT[act],
                                None if bg is None else dev(gpu, bg), None if bu is None else dev(gpu, bu), cfg)
    gpu.cuda.synchronize()
    got = got.cpu().numpy()
    want = oracle.c_gated_ffn(t, x, Wg, Wu, bg, bu, act, norm)
    # scale of the product of the two contractions: the error of either factor is bounded on its own
    # contraction's scale, so the product is judged on max|gate| * max|up| (pre-activation for the gate)
    xn = x if norm is None else oracle.c_rmsnorm(x, *norm)
    g_pre, g_act = oracle.c_qdense(t, xn, Wg, bg, 0), oracle.c_qdense(t, xn, Wg, bg, act)
    up = oracle.c_qdense(t, xn, Wu, bu, 0)
    scale = max(float(np.max(np.abs(g_pre))), float(np.max(np.abs(g_act)))) * float(np.max(np.abs(up))) or 1.0
    err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) / scale
    assert got.shape == (M, N) and np.all(np.isfinite(got))
    return err


def test_gemm_epilogues_stay_inside_their_output(gpu, oracle):
    """The GEMM kernels write whole interior tiles without per-element bounds checks.  Outputs placed in the middle of a
    larger buffer filled with a sentinel: shapes that are exact multiples of the tiles, one row / column over and under,
    and a gated pair whose interleaved weight image is longer than twice its outputs - the sentinel on both sides must
    survive and the result must be right."""
    import ctypes
    from gomlx_amd import _lib
    L = _lib.lib()
    stream = gpu.cuda.current_stream().cuda_stream
    pad = 4096
    t = Q8_0
    for M, K, N, bf16 in [(256, 512, 128, True), (512, 512, 256, False), (257, 512, 129, True), (255, 512, 127, False), (1408, 256, 192, True),
                          (384, 512, 320, False)]:
        W, x = synth.weights(t, 9500 + M, N, K), synth.activations(9501 + N, M, K)
        xin = bf16_round(x) if bf16 else x
        buf = gpu.full((pad + M * N + pad,), 12345.0, device="cuda")
        xd = dev(gpu, xin).to(gpu.bfloat16) if bf16 else dev(gpu, xin)
        Wd = dev(gpu, W)  # (kept alive until the call has run)
        fn = L.gq_qdense_bf16 if bf16 else L.gq_qdense_f32
        _lib.check(fn(t, xd.data_ptr(), M, K, Wd.data_ptr(), N, None, 0, buf.data_ptr() + 4 * pad, stream))
        gpu.cuda.synchronize()
        h = buf.cpu().numpy()
        assert np.all(h[:pad] == 12345.0) and np.all(h[pad + M * N:] == 12345.0), (M, K, N, bf16)
        assert rel_err(h[pad:pad + M * N].reshape(M, N), oracle.c_qdense(t, xin, W)) < (TOL_BF16 if bf16 else TOL_F32)
    for M, K, N in [(256, 512, 1000), (512, 256, 64), (300, 512, 96)]:
        Wg, Wu, x = synth.weights(t, 9600 + N, N, K), synth.weights(t, 9601 + N, N, K), synth.activations(9602 + M, M, K)
        buf = gpu.full((pad + M * N + pad,), 12345.0, device="cuda")
        xd, Wgd, Wud = dev(gpu, x), dev(gpu, Wg), dev(gpu, Wu)
        _lib.check(L.gq_qdense_gated_f32(t, xd.data_ptr(), M, K, None, Wgd.data_ptr(), None, Wud.data_ptr(), None, N, 3,
                                         buf.data_ptr() + 4 * pad, stream))
        gpu.cuda.synchronize()
        h = buf.cpu().numpy()
        assert np.all(h[:pad] == 12345.0) and np.all(h[pad + M * N:] == 12345.0), ("gated", M, K, N)
        want = oracle.c_gated_ffn(t, x, Wg, Wu, None, None, 3, None)
        scale = float(np.max(np.abs(oracle.c_qdense(t, x, Wg)))) * float(np.max(np.abs(oracle.c_qdense(t, x, Wu))))
        assert float(np.max(np.abs(h[pad:pad + M * N].reshape(M, N).astype(np.float64) - want))) / scale < 2 * TOL_F32


@pytest.mark.parametrize("t", ALL_TYPES)
def test_gated_feed_forward_decode(gpu, oracle, t):
    """Fused path: up to 16 rows, K a multiple of 256 (one launch over both matrices)."""
    for i, (M, K, N, act, norm_kind, with_bias) in enumerate([
            (1, 4096, 1000, 3, 1, False), (1, 512, 8, 3, 0, False), (2, 2304, 333, 1, 2, True), (1, 256, 1, 3, 3, True),
            (4, 1536, 130, 5, 1, True), (16, 1024, 70, 3, 2, False), (1, 4608, 64, 2, 0, True), (3, 768, 1030, 4, 3, False)]):
        err = gated_case(gpu, oracle, t, M, K, N, act, norm_kind, with_bias, 400 + 10 * i + t)
        assert err < 2 * TOL_F32, (t, M, K, N, act, norm_kind, with_bias, err)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_gated_feed_forward_composed(gpu, oracle, t):
    """Shapes outside the fused path (more rows, ragged K for the 32-value formats) are composed of
    dense calls; those from 17 rows on contract fp16 operands."""
    ragged_k = 160 if t in (Q4_0, Q8_0, IQ4_NL) else 768
    for i, (M, K, N, act, norm_kind, with_bias) in enumerate([
            (17, 1024, 96, 3, 1, True), (40, 512, 256, 3, 0, False), (2, ragged_k, 50, 3, 2, True),
            (130, 1024, 128, 1, 1, False)]):
        err = gated_case(gpu, oracle, t, M, K, N, act, norm_kind, with_bias, 600 + 10 * i + t)
        assert err < 2 * TOL_F32, (t, M, K, N, act, norm_kind, with_bias, err)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_dense_with_rmsnorm_and_residual(gpu, oracle, t):
    """y = residual + act(RMSNorm(x) . W^T + b): norm alone, residual alone, both; fused shapes (up to 16
    rows, K % 256 == 0) and composed ones; the residual updated in place."""
    for i, (M, K, N, act, use_norm, use_res) in enumerate([
            (1, 4096, 512, 0, True, False), (3, 768, 100, 3, True, True), (16, 256, 33, 0, False, True), (20, 512, 64, 0, True, True),
            (1, 2304, 1, 5, True, False), (40, 1024, 128, 0, False, True), (2, 4608, 70, 1, True, True)]):
        W = synth.weights(t, 700 + i, N, K)
        x = (synth.activations(701 + i, M, K) * 3.0).astype(np.float32)
        gain = (synth.normal(702 + i, 0, K) * 0.5 + 1.0).astype(np.float32)
        bias = synth.normal(703 + i, 0, N).astype(np.float32) * 0.1
        res = synth.activations(704 + i, M, N)
        rd = dev(gpu, res) if use_res else None
        got = nn.quantized_dense(dev(gpu, x), dev(gpu, W), Quantization(ggml_type=t), dev(gpu, bias), BACKEND_ACT[act],
                                 norm=nn.RMSNorm(dev(gpu, gain), 1e-6, 0.0) if use_norm else None, residual=rd).cpu().numpy()
        xn = oracle.c_rmsnorm(x, gain, 1e-6, 0.0) if use_norm else x
        dense = oracle.c_qdense(t, xn, W, bias, act)
        want = dense + res if use_res else dense
        pre = oracle.c_qdense(t, xn, W, bias, 0)
        scale = max(float(np.max(np.abs(dense))), float(np.max(np.abs(pre))))
        err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) / scale
        assert err < TOL_F32, (t, M, K, N, act, use_norm, use_res, err)
    # in place: y is the residual buffer itself
    import ctypes
    from gomlx_amd import _lib
    M, K, N = 2, 512, 96
    W, x, res = synth.weights(t, 720, N, K), synth.activations(721, M, K), synth.activations(722, M, N)
    xd, Wd, yd = dev(gpu, x), dev(gpu, W), dev(gpu, res)
    _lib.check(_lib.lib().gq_qdense_block_f32(t, xd.data_ptr(), M, K, None, Wd.data_ptr(), N, None, 0, yd.data_ptr(), yd.data_ptr(),
                                              gpu.cuda.current_stream().cuda_stream))
    gpu.cuda.synchronize()
    assert rel_err(yd.cpu().numpy(), oracle.c_qdense(t, x, W) + res) < TOL_F32


# Bounds of the per-element form |got - want| <= tol * rms(want), by route.  For Gaussian outputs max|want| is 3.5 to
# 4.5 times rms(want), so this form is that much stricter than the max-norm metric above.  The integer-dot GEMV keeps
# fp32-path accuracy with a wide margin; the routes that contract fp32 activations on the matrix cores round x (split-K)
# or x and W (two passes) to fp16 operands, which puts them at about the 1e-3 mark in this form: they are the MFMA class of
# the accuracy statement (2e-2), and are held here to a bound an order of magnitude tighter than that.
RMS_TOL = {"gemv": 1e-3, "split-k": 3e-3, "two-pass f32": 4e-3, "bf16": 2e-2}


def test_error_scaled_by_rms_per_route(gpu, oracle):
    # (a matrix this small stays on GEMV passes for every batch of up to 16 rows: the split-K rows start at 17)
    K, N = 4096, 512
    worst = {}
    for t in ALL_TYPES:
        W = synth.weights(t, 8100 + t, N, K)
        for route, M, bf16 in (("gemv", 1, False), ("gemv", 4, False), ("gemv", 8, False), ("split-k", 17, False), ("split-k", 32, False), ("two-pass f32", 256, False),
                               ("bf16", 32, True), ("bf16", 256, True)):
            x = synth.activations(8200 + M, M, K)
            want = oracle.c_qdense(t, bf16_round(x) if bf16 else x, W)
            got = run_dense(gpu, t, x, W, None, 0, bf16=bf16)
            e = rms_err(got, want)
            rel_err(got, want)
            worst[route] = max(worst.get(route, 0.0), e)
            assert e < RMS_TOL[route], (ggml.name(t), route, M, e)
    print("max|d| / rms(want) by route:", {k: f"{v:.2e}" for k, v in worst.items()})


# Rounding units of the operands each route contracts (u_x for the activations, u_w for the weights), for the standard
# forward bound of a dot product whose operands are rounded first: |got - want| <= (u_x + u_w) * sum_k |x_k| |w_k| (plus
# the fp32 accumulation, orders of magnitude below).  The decode GEMV rounds x to 16-bit fixed point relative to the
# largest value of its 32-value block (so its x term is taken against the block maxima) and keeps W exact; the split-K
# kernels and the fp32 two-pass route round x (after a power-of-two scaling per row) and W to fp16; the bf16 routes take x
# as given and round W to bf16 (8 significant bits: half a unit in the last place is 2^-8).
OPERAND_ROUNDING = {"gemv": (2.0 ** -16, 0.0), "split-k": (2.0 ** -11, 2.0 ** -11), "two-pass f32": (2.0 ** -11, 2.0 ** -11), "bf16": (0.0, 2.0 ** -8)}


@pytest.mark.parametrize("scale", [1e3, 1e5])
def test_heavy_tailed_activations_per_route(gpu, oracle, scale):
    """The activations a decoder produces: a few channels hundreds to many thousands of times the rest (four of the K
    channels scaled by 1e3 or 1e5, the same ones in every row, as the outlier features of real models are).  Four terms then
    carry every output, so operand rounding no longer averages out over K as it does for Gaussian inputs, and a block or a
    row that holds an outlier loses its small values' low bits.  Checked three ways: the max-norm bound of the accuracy
    statement (1e-3 for fp32 activations, 2e-2 for bf16) must hold as for any input; every ELEMENT must be within the
    forward bound that the route's operand rounding allows, (u_x + u_w) * sum_k |x_k w_k| with 25 % slack (values more than
    2^23 below the largest of their row and K-slice fall into fp16's subnormal range, where the rounding is absolute) - an
    error beyond that would be a defect of the kernel, not of its operand format; and the per-element form against rms(want) is printed
    (it reads up to 3e-2 for the bf16 routes here: bf16 weights, four terms)."""
    K, N = 4096, 512
    hot = [5, 1000, 2049, 4000]
    worst, used = {}, {}
    for t in ALL_TYPES:
        W = synth.weights(t, 8400 + t, N, K)
        absW = np.abs(oracle.c_dequantize(t, W, K).astype(np.float64))
        for route, M, bf16 in (("gemv", 1, False), ("gemv", 4, False), ("gemv", 8, False), ("split-k", 17, False), ("split-k", 32, False), ("two-pass f32", 256, False),
                               ("bf16", 32, True), ("bf16", 256, True)):
            x = synth.activations(8500 + M, M, K)
            x[:, hot] *= np.float32(scale)
            xin = bf16_round(x) if bf16 else x
            want = oracle.c_qdense(t, xin, W)
            got = run_dense(gpu, t, x, W, None, 0, bf16=bf16)
            assert rel_err(got, want) < (TOL_BF16 if bf16 else TOL_F32), (ggml.name(t), route, M, scale)
            worst[route] = max(worst.get(route, 0.0), rms_err(got, want))
            ax = np.abs(xin.astype(np.float64))
            ux, uw = OPERAND_ROUNDING[route]
            if route == "gemv":  # fixed point relative to the block's largest value
                ax_round = np.repeat(ax.reshape(M, K // 32, 32).max(axis=2), 32, axis=1)
            else:
                ax_round = ax
            bound = ux * (ax_round @ absW.T) + (uw + 2.0 ** -21) * (ax @ absW.T)
            frac = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)) / bound))
            used[route] = max(used.get(route, 0.0), frac)
            assert frac < 1.25, (ggml.name(t), route, M, scale, frac)
    print(f"outliers x {scale:g}: max|d| / rms(want) by route:", {k: f"{v:.2e}" for k, v in worst.items()},
          "; largest share of the operand-rounding bound used by an element:", {k: f"{v:.2f}" for k, v in used.items()})


@pytest.mark.parametrize("t", ALL_TYPES)
def test_callers_around_a_projection_with_bf16_activations(gpu, oracle, t):
    """RMSNorm + projection + residual, q/k/v behind one norm, and the gated feed-forward front for bf16 activations:
    bit-identical to the fp32 entry points on the widened inputs (the widening is exact), and within the fp32-path
    bound of the oracle on the bf16-rounded inputs; decode rows, split-K batches and a two-pass batch."""
    q = Quantization(ggml_type=t)
    for i, (M, K, N, act) in enumerate([(1, 4096, 384, 0), (3, 1024, 200, 3), (24, 2048, 260, 0), (200, 1024, 128, 1)]):
        x32 = bf16_round((synth.activations(8300 + i, M, K) * 2.5).astype(np.float32))
        xb = dev(gpu, x32).to(gpu.bfloat16)
        gain = (synth.normal(8310 + i, 0, K) * 0.5 + 1.0).astype(np.float32)
        bias = synth.normal(8320 + i, 0, N).astype(np.float32) * 0.1
        res = synth.activations(8330 + i, M, N)
        W, W2 = synth.weights(t, 8340 + i, N, K), synth.weights(t, 8350 + i, N, K)
        norm = nn.RMSNorm(dev(gpu, gain), 1e-6, 0.0)
        xn = oracle.c_rmsnorm(x32, gain, 1e-6, 0.0)
        # projection with norm and residual
        got = nn.quantized_dense(xb, dev(gpu, W), q, dev(gpu, bias), BACKEND_ACT[act], norm=norm, residual=dev(gpu, res)).cpu().numpy()
        same = nn.quantized_dense(dev(gpu, x32), dev(gpu, W), q, dev(gpu, bias), BACKEND_ACT[act], norm=norm, residual=dev(gpu, res)).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), same.view(np.uint32)), (ggml.name(t), M, K, N)
        dense, pre = oracle.c_qdense(t, xn, W, bias, act), oracle.c_qdense(t, xn, W, bias, 0)
        scale = max(float(np.max(np.abs(dense))), float(np.max(np.abs(pre))))
        tol = TOL_F32 if M <= 192 else 2 * TOL_F32
        assert float(np.max(np.abs(got.astype(np.float64) - (dense + res)))) / scale < tol, (ggml.name(t), M, K, N)
        # gated feed-forward front
        got = nn.gated_feed_forward(xb, dev(gpu, W), dev(gpu, W2), q, Activation.SILU, dev(gpu, bias), None, norm=norm).cpu().numpy()
        same = nn.gated_feed_forward(dev(gpu, x32), dev(gpu, W), dev(gpu, W2), q, Activation.SILU, dev(gpu, bias), None, norm=norm).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), same.view(np.uint32)), ("gated", ggml.name(t), M, K, N)
        gate, up = oracle.c_qdense(t, xn, W, bias, 0), oracle.c_qdense(t, xn, W2, None, 0)
        want = oracle.c_qdense(t, xn, W, bias, 3).astype(np.float64) * up
        assert float(np.max(np.abs(got - want))) / (float(np.max(np.abs(gate))) * float(np.max(np.abs(up)))) < 2 * tol, ("gated", ggml.name(t), M, K, N)
        # q / k / v behind one norm: one shared activation matrix, widened once
        if M <= 8:
            probs = [(xb, dev(gpu, W), q, None, None), (xb, dev(gpu, W2), q, dev(gpu, bias), None), (xb, dev(gpu, W[: N // 2]), q, None, None)]
            outs = nn.quantized_dense_batch(probs, norm=norm)
            x32d = dev(gpu, x32)
            same = nn.quantized_dense_batch([(x32d,) + p[1:] for p in probs], norm=norm)
            for out, ref, (Wm, b) in zip(outs, same, ((W, None), (W2, bias), (W[: N // 2], None))):
                assert gpu.equal(out, ref), ("batch", ggml.name(t), M, K, N)
                assert rel_err(out.cpu().numpy(), oracle.c_qdense(t, xn, Wm, b, 0)) < TOL_F32
            # a normalisation without a learned scale, and a residual without a normalisation: the decode kernel reads
            # the bf16 rows as they are (no gain to fetch beside them)
            plain = nn.RMSNorm(None, 1e-5, 0.0)
            for kw in (dict(norm=plain), dict(residual=dev(gpu, res)), dict(norm=plain, residual=dev(gpu, res))):
                got = nn.quantized_dense(xb, dev(gpu, W), q, None, BACKEND_ACT[act], **kw)
                ref = nn.quantized_dense(x32d, dev(gpu, W), q, None, BACKEND_ACT[act], **kw)
                assert gpu.equal(got, ref), (sorted(kw), ggml.name(t), M, K, N)
            xp = oracle.c_rmsnorm(x32, np.ones(K, np.float32), 1e-5, 0.0)
            got = nn.quantized_dense(xb, dev(gpu, W), q, None, norm=plain, residual=dev(gpu, res)).cpu().numpy()
            dense = oracle.c_qdense(t, xp, W, None, 0)
            assert float(np.max(np.abs(got.astype(np.float64) - (dense + res)))) / float(np.max(np.abs(dense))) < TOL_F32, (ggml.name(t), M, K, N)
            got = nn.gated_feed_forward(xb, dev(gpu, W), dev(gpu, W2), q, Activation.SILU, None, None, norm=plain)
            ref = nn.gated_feed_forward(x32d, dev(gpu, W), dev(gpu, W2), q, Activation.SILU, None, None, norm=plain)
            assert gpu.equal(got, ref), ("gated, no scale", ggml.name(t), M, K, N)


@pytest.mark.parametrize("t,M,K,N", [(Q4_K, 2, 4096, 14336), (Q4_K, 3, 4096, 14336), (Q8_0, 2, 4096, 8192), (Q4_0, 1, 1280, 300),
                                     (Q6_K, 2, 1280, 264), (IQ4_NL, 5, 2304, 128), (Q4_K, 16, 1024, 64)])
def test_bf16_rows_in_the_decode_kernel_with_its_extras(gpu, oracle, t, M, K, N):
    """bf16 activations read by the decode kernel itself, with normalisation, gated product and residual: passes of two rows
    over a large matrix, a K that ends in a half slice, several rows over a small matrix.  Bit-identical to the fp32 entry
    points on the widened inputs and within the fp32 bound of the oracle."""
    q = Quantization(ggml_type=t)
    x32 = bf16_round((synth.activations(8400 + M, M, K) * 1.5).astype(np.float32))
    xb, xw = dev(gpu, x32).to(gpu.bfloat16), dev(gpu, x32)
    gain = (synth.normal(8410, 0, K) * 0.5 + 1.0).astype(np.float32)
    res = synth.activations(8420, M, N)
    W, W2 = synth.weights(t, 8430, N, K), synth.weights(t, 8431, N, K)
    Wd, W2d, resd = dev(gpu, W), dev(gpu, W2), dev(gpu, res)
    for norm, gain_h in ((nn.RMSNorm(dev(gpu, gain), 1e-6, 1.0), gain + 1.0), (nn.RMSNorm(None, 1e-6, 0.0), np.ones(K, np.float32))):
        got = nn.quantized_dense(xb, Wd, q, None, norm=norm, residual=resd)
        assert gpu.equal(got, nn.quantized_dense(xw, Wd, q, None, norm=norm, residual=resd)), (ggml.name(t), M, K, N)
        xn = oracle.c_rmsnorm(x32, gain_h, 1e-6, 0.0)
        dense = oracle.c_qdense(t, xn, W, None, 0)
        assert float(np.max(np.abs(got.cpu().numpy().astype(np.float64) - (dense + res)))) / float(np.max(np.abs(dense))) < TOL_F32
        got = nn.gated_feed_forward(xb, Wd, W2d, q, Activation.SILU, None, None, norm=norm)
        assert gpu.equal(got, nn.gated_feed_forward(xw, Wd, W2d, q, Activation.SILU, None, None, norm=norm)), ("gated", ggml.name(t), M, K, N)
        gate, up = oracle.c_qdense(t, xn, W, None, 0), oracle.c_qdense(t, xn, W2, None, 0)
        want = oracle.c_qdense(t, xn, W, None, 3).astype(np.float64) * up
        assert float(np.max(np.abs(got.cpu().numpy() - want))) / (float(np.max(np.abs(gate))) * float(np.max(np.abs(up)))) < 2 * TOL_F32


def test_residual_in_place_on_the_composed_path(gpu, oracle):
    """y == residual on shapes that none of the fused routes take (K not a multiple of 256; N not a multiple of 4
    beyond 16 rows): the dense result must not overwrite the residual before it is added."""
    from gomlx_amd import _lib
    L = _lib.lib()
    stream = gpu.cuda.current_stream().cuda_stream
    for i, (t, M, K, N, use_norm) in enumerate([(Q8_0, 2, 160, 64, False), (Q8_0, 20, 160, 33, False), (Q4_0, 20, 512, 33, True),
                                               (Q4_K, 24, 768, 30, False), (Q8_0, 3, 96, 10, True)]):
        W, x, res = synth.weights(t, 730 + i, N, K), synth.activations(740 + i, M, K), synth.activations(750 + i, M, N)
        gain = (synth.normal(760 + i, 0, K) * 0.5 + 1.0).astype(np.float32)
        xd, Wd, yd, gd = dev(gpu, x), dev(gpu, W), dev(gpu, res), dev(gpu, gain)
        norm = _lib.RmsNormDesc(gd.data_ptr(), 1e-6, 0.0)
        import ctypes
        _lib.check(L.gq_qdense_block_f32(t, xd.data_ptr(), M, K, ctypes.byref(norm) if use_norm else None, Wd.data_ptr(), N, None, 0,
                                         yd.data_ptr(), yd.data_ptr(), stream))
        gpu.cuda.synchronize()
        xn = oracle.c_rmsnorm(x, gain, 1e-6, 0.0) if use_norm else x
        dense = oracle.c_qdense(t, xn, W)
        err = float(np.max(np.abs(yd.cpu().numpy().astype(np.float64) - (dense + res)))) / float(np.max(np.abs(dense)))
        assert err < TOL_F32, (ggml.name(t), M, K, N, use_norm, err)


def test_two_host_threads_share_the_null_stream(gpu, oracle):
    """Split-K calls (three kernels that share the stream's workspace) issued concurrently from two host threads on the
    null stream: every result matches the oracle, i.e. the launch sequences were not interleaved."""
    import threading
    from gomlx_amd import _lib
    L = _lib.lib()
    t, M, K, N = Q4_K, 32, 2048, 512
    jobs = []
    for i in range(2):
        W, x = synth.weights(t, 7800 + i, N, K), synth.activations(7810 + i, M, K) * (1.0 + 3.0 * i)
        jobs.append(dict(W=W, x=x.astype(np.float32), Wd=dev(gpu, W), xd=dev(gpu, x.astype(np.float32)),
                         ys=[gpu.zeros((M, N), device="cuda") for _ in range(40)], rc=[]))
    gpu.cuda.synchronize()
    start = threading.Barrier(2)

    def work(j):
        start.wait()
        for y in j["ys"]:
            j["rc"].append(L.gq_qdense_f32(t, j["xd"].data_ptr(), M, K, j["Wd"].data_ptr(), N, None, 0, y.data_ptr(), None))

    threads = [threading.Thread(target=work, args=(j,)) for j in jobs]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    gpu.cuda.synchronize()
    for j in jobs:
        assert all(rc == 0 for rc in j["rc"])
        want = oracle.c_qdense(t, j["x"], j["W"])
        for y in j["ys"]:
            assert rel_err(y.cpu().numpy(), want) < TOL_F32


def test_graph_replays_only_on_its_recording_stream(gpu):
    import ctypes
    from gomlx_amd import _lib
    L = _lib.lib()
    t, M, K, N = Q8_0, 8, 1024, 256
    W, x = dev(gpu, synth.weights(t, 7900, N, K)), dev(gpu, synth.activations(7901, M, K))
    y = gpu.zeros((M, N), device="cuda")
    s1, s2 = gpu.cuda.Stream(), gpu.cuda.Stream()
    _lib.check(L.gq_qdense_f32(t, x.data_ptr(), M, K, W.data_ptr(), N, None, 0, y.data_ptr(), s1.cuda_stream))
    gpu.cuda.synchronize()
    _lib.check(L.gq_graph_begin(s1.cuda_stream))
    _lib.check(L.gq_qdense_f32(t, x.data_ptr(), M, K, W.data_ptr(), N, None, 0, y.data_ptr(), s1.cuda_stream))
    g = ctypes.c_void_p()
    _lib.check(L.gq_graph_end(s1.cuda_stream, ctypes.byref(g)))
    assert L.gq_graph_launch(g, s2.cuda_stream) == _lib.ERR_INVALID
    _lib.check(L.gq_graph_launch(g, s1.cuda_stream))
    gpu.cuda.synchronize()
    _lib.check(L.gq_graph_destroy(g))


@pytest.mark.parametrize("t", ALL_TYPES)
def test_split_k_batches_carry_the_normalisation(gpu, oracle, t):
    """In the split-K range the gain is applied where the activation image is written and the division by the root
    mean square in the reduction over K-slices (one to sixteen slices here): with and without gain, with a gain
    offset, a large epsilon, a residual, the gated product, and a gain whose address is not 16-byte aligned (which
    takes the separate normalisation kernel)."""
    q = Quantization(ggml_type=t)
    cases = [(17, 512, 132, 1, 1e-6, 0.0, True, False), (33, 1024, 512, 0, 1e-2, 0.0, False, False), (96, 2560, 64, 1, 1e-5, 1.0, True, False),
             (20, 4096, 260, 1, 1e-6, 0.0, False, True), (64, 8192, 36, 2, 1e-6, 0.0, True, False), (24, 1536, 128, 1, 1e-5, 1.0, False, True)]
    for i, (M, K, N, gain_kind, eps, off, use_res, gated) in enumerate(cases):
        x = (synth.activations(771 + i, M, K) * 4.0).astype(np.float32)
        gain = (synth.normal(772 + i, 0, K + 1) * 0.5 + 1.0 - off).astype(np.float32)
        gd = dev(gpu, gain)
        g_host, g_dev = (None, None) if gain_kind == 0 else (gain[:K], gd[:K]) if gain_kind == 1 else (gain[1:], gd[1:])
        cfg = nn.RMSNorm(g_dev, eps, off)
        xn = oracle.c_rmsnorm(x, g_host, eps, off)
        W = synth.weights(t, 773 + i, N, K)
        bias = synth.normal(774 + i, 0, N).astype(np.float32) * 0.1
        if gated:
            W2 = synth.weights(t, 775 + i, N, K)
            got = nn.gated_feed_forward(dev(gpu, x), dev(gpu, W), dev(gpu, W2), q, Activation.SILU, dev(gpu, bias), None, norm=cfg).cpu().numpy()
            gate, up = oracle.c_qdense(t, xn, W, bias, 0), oracle.c_qdense(t, xn, W2, None, 0)
            want = oracle.c_qdense(t, xn, W, bias, 3).astype(np.float64) * up
            err = float(np.max(np.abs(got - want))) / (float(np.max(np.abs(gate))) * float(np.max(np.abs(up))))
            assert err < 2 * TOL_F32, ("gated", t, M, K, N, err)
            continue
        res = synth.activations(776 + i, M, N)
        got = nn.quantized_dense(dev(gpu, x), dev(gpu, W), q, dev(gpu, bias), Activation.NONE, norm=cfg,
                                 residual=dev(gpu, res) if use_res else None).cpu().numpy()
        dense = oracle.c_qdense(t, xn, W, bias, 0)
        want = dense + res if use_res else dense
        err = float(np.max(np.abs(got.astype(np.float64) - want))) / float(np.max(np.abs(dense)))
        assert err < TOL_F32, (t, M, K, N, gain_kind, eps, off, use_res, err)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_batched_projections_behind_one_norm(gpu, oracle, t):
    """q/k/v of a layer: three batch-1 projections of one normalised input in one launch; a list that
    cannot be merged (a batch of 3 rows among them) gives the same results through separate calls."""
    K = 2048
    gain = (synth.normal(740, 0, K) * 0.5 + 1.0).astype(np.float32)
    cfg = nn.RMSNorm(dev(gpu, gain), 1e-5, 0.0)
    q = Quantization(ggml_type=t)
    for rows in ((1, 1, 1), (1, 3, 1), (4, 4, 4), (8, 8, 8), (9, 9, 9)):  # (up to 8 rows each share the launch too)
        xs = [synth.activations(741 + j, m, K) for j, m in enumerate(rows)]
        if len(set(rows)) == 1:
            xs = [xs[0]] * 3  # one shared input, as in a decoder layer
        Ws = [synth.weights(t, 750 + j, n, K) for j, n in enumerate((2048, 512, 520))]
        bs = [None, synth.normal(760, 0, 512).astype(np.float32) * 0.1, None]
        outs = nn.quantized_dense_batch([(dev(gpu, x), dev(gpu, W), q, None if b is None else dev(gpu, b), None)
                                         for x, W, b in zip(xs, Ws, bs)], norm=cfg)
        gpu.cuda.synchronize()
        for x, W, b, y in zip(xs, Ws, bs, outs):
            want = oracle.c_qdense(t, oracle.c_rmsnorm(x, gain, 1e-5, 0.0), W, b)
            assert rel_err(y.cpu().numpy(), want) < TOL_F32
        plain = nn.quantized_dense_batch([(dev(gpu, x), dev(gpu, W), q, None if b is None else dev(gpu, b), None)
                                          for x, W, b in zip(xs, Ws, bs)])
        gpu.cuda.synchronize()
        for x, W, b, y in zip(xs, Ws, bs, plain):
            assert rel_err(y.cpu().numpy(), oracle.c_qdense(t, x, W, b)) < TOL_F32


@pytest.mark.parametrize("t", ALL_TYPES)
def test_projections_of_one_input_share_the_two_passes(gpu, oracle, t):
    """q / k / v past the split-K range: the activations are normalised and converted once, the matrices' 16-bit images
    follow each other and ONE GEMM writes each matrix's columns to its own output (widths that are multiples of 32, one
    activation for all, each with or without bias).  Checked against the oracle; row counts on and off the tiles, two to
    four matrices; a width that is not a multiple of 32 and mixed activations take the separate calls."""
    K = 1024
    gain = (synth.normal(1770, 0, K) * 0.5 + 1.0).astype(np.float32)
    cfg = nn.RMSNorm(dev(gpu, gain), 1e-5, 0.0)
    q = Quantization(ggml_type=t)
    widths = (512, 128, 96, 64)
    Ws = [synth.weights(t, 1772 + j, n, K) for j, n in enumerate(widths)]
    bs = [None, synth.normal(1775, 0, 128).astype(np.float32) * 0.1, None, synth.normal(1776, 0, 64).astype(np.float32) * 0.1]
    for rows in (130, 256, 300):
        x = synth.activations(1771 + rows, rows, K)
        xd = dev(gpu, x)
        xn = oracle.c_rmsnorm(x, gain, 1e-5, 0.0)
        for count in (3, 2, 4):
            outs = nn.quantized_dense_batch([(xd, dev(gpu, W), q, None if b is None else dev(gpu, b), None) for W, b in zip(Ws[:count], bs)], norm=cfg)
            gpu.cuda.synchronize()
            for W, b, y in zip(Ws, bs, outs):
                assert rel_err(y.cpu().numpy(), oracle.c_qdense(t, xn, W, b)) < TOL_F32, (ggml.name(t), rows, count, W.shape)
    # one activation for all: SiLU
    outs = nn.quantized_dense_batch([(xd, dev(gpu, W), q, None, BACKEND_ACT[3]) for W in Ws[:3]], norm=cfg)
    for W, y in zip(Ws, outs):
        assert rel_err(y.cpu().numpy(), oracle.c_qdense(t, xn, W, None, 3)) < TOL_F32
    # outside the shared form: a width of 100, and mixed activations
    odd = synth.weights(t, 1790, 100, K)
    outs = nn.quantized_dense_batch([(xd, dev(gpu, Ws[0]), q, None, None), (xd, dev(gpu, odd), q, None, None)], norm=cfg)
    assert rel_err(outs[1].cpu().numpy(), oracle.c_qdense(t, xn, odd, None)) < TOL_F32
    outs = nn.quantized_dense_batch([(xd, dev(gpu, Ws[0]), q, None, None), (xd, dev(gpu, Ws[1]), q, None, BACKEND_ACT[2])], norm=cfg)
    assert rel_err(outs[1].cpu().numpy(), oracle.c_qdense(t, xn, Ws[1], None, 2)) < TOL_F32
    # bf16 activations behind the normalisation: widened exactly, then the same route
    xb = bf16_round(x)
    outs = nn.quantized_dense_batch([(dev(gpu, xb).to(gpu.bfloat16), dev(gpu, W), q, None, None) for W in Ws[:3]], norm=cfg)
    same = nn.quantized_dense_batch([(dev(gpu, xb), dev(gpu, W), q, None, None) for W in Ws[:3]], norm=cfg)
    for y, ref in zip(outs, same):
        assert gpu.equal(y, ref)


@pytest.mark.parametrize("rows,K", [(6, 2048), (8, 4096), (12, 2048), (32, 4096), (70, 2048), (33, 1536)])
def test_projections_of_one_input_share_a_split_k_pass(gpu, oracle, rows, K):
    """q / k / v beyond the GEMV's rows: three Q4_K projections of ONE device buffer of activations behind one normalisation
    (one activation image, one main launch over all rows, one reduction), each with its own width, bias and activation; the
    same list without the normalisation, and with distinct inputs, goes through separate calls."""
    t = Q4_K
    gain = (synth.normal(770, 0, K) * 0.5 + 1.0).astype(np.float32)
    cfg = nn.RMSNorm(dev(gpu, gain), 1e-5, 0.0)
    q = Quantization(ggml_type=t)
    x = synth.activations(771, rows, K)
    xd = dev(gpu, x)
    Ws = [synth.weights(t, 772 + j, n, K) for j, n in enumerate((2048, 512, 260))]
    bs = [None, synth.normal(775, 0, 512).astype(np.float32) * 0.1, synth.normal(776, 0, 260).astype(np.float32) * 0.1]
    acts = [0, 3, 0]
    outs = nn.quantized_dense_batch([(xd, dev(gpu, W), q, None if b is None else dev(gpu, b), BACKEND_ACT[a])
                                     for W, b, a in zip(Ws, bs, acts)], norm=cfg)
    gpu.cuda.synchronize()
    xn = oracle.c_rmsnorm(x, gain, 1e-5, 0.0)
    for W, b, a, y in zip(Ws, bs, acts, outs):
        assert rel_err(y.cpu().numpy(), oracle.c_qdense(t, xn, W, b, a)) < TOL_F32, (rows, K, W.shape)
    # two projections only, and a fourth
    more = Ws + [synth.weights(t, 779, 128, K)]
    for count in (2, 4):
        outs = nn.quantized_dense_batch([(xd, dev(gpu, W), q, None, None) for W in more[:count]], norm=cfg)
        gpu.cuda.synchronize()
        for W, y in zip(more, outs):
            assert rel_err(y.cpu().numpy(), oracle.c_qdense(t, xn, W, None)) < TOL_F32, (rows, K, count, W.shape)
    # the same list without a normalisation (gq_qdense_f32_batch)
    outs = nn.quantized_dense_batch([(xd, dev(gpu, W), q, None if b is None else dev(gpu, b), BACKEND_ACT[a])
                                     for W, b, a in zip(Ws, bs, acts)])
    gpu.cuda.synchronize()
    for W, b, a, y in zip(Ws, bs, acts, outs):
        assert rel_err(y.cpu().numpy(), oracle.c_qdense(t, x, W, b, a)) < TOL_F32, (rows, K, W.shape, "no norm")
    # bf16 activations behind the normalisation: the pre-pass widens them (exact), the same pass
    xb = bf16_round(x)
    xbd = dev(gpu, xb).to(gpu.bfloat16)
    outs = nn.quantized_dense_batch([(xbd, dev(gpu, W), q, None, None) for W in Ws], norm=cfg)
    gpu.cuda.synchronize()
    xbn = oracle.c_rmsnorm(xb, gain, 1e-5, 0.0)
    xb32 = dev(gpu, xb)  # (one buffer: the list shares a pass only as projections of the same activations)
    same = nn.quantized_dense_batch([(xb32, dev(gpu, W), q, None, None) for W in Ws], norm=cfg)
    for W, y, ref in zip(Ws, outs, same):
        assert gpu.equal(y, ref), (rows, K, "bf16 against the widened input")
        assert rel_err(y.cpu().numpy(), oracle.c_qdense(t, xbn, W, None)) < TOL_F32, (rows, K, "bf16")


def test_batched_submissions_randomized(gpu, oracle):
    """Seeded random lists of two to eight projections of one format and one to three rows, through gq_qdense_f32_batch and
    (one K, fp32 or bf16 activations) behind a shared normalisation: widths from a single row to a few thousand, K with and
    without a half slice and with more slices than wavefronts, so that the workgroups of one launch own anything from one
    row-step (padded to the kernel's group of two) to dozens."""
    rng = np.random.default_rng(20240611)
    for case in range(24):
        t = ALL_TYPES[int(rng.integers(len(ALL_TYPES)))]
        q = Quantization(ggml_type=t)
        count, rows = int(rng.integers(2, 9)), int(rng.choice([1, 1, 1, 2, 3]))
        use_norm = bool(rng.integers(2))
        bf16 = use_norm and bool(rng.integers(2))
        same_k = int(rng.choice([256, 768, 1024, 1280, 2048, 3584, 4608, 5120, 6144, 8192, 14336]))
        gain = (synth.normal(9100 + case, 0, same_k) * 0.5 + 1.0).astype(np.float32)
        norm = nn.RMSNorm(dev(gpu, gain), 1e-5, 0.0) if use_norm else None
        hosts, probs = [], []
        for i in range(count):
            K = same_k if use_norm else int(rng.choice([256, 512, 1024, 1280, 2048, 4096, 5120, 14336]))
            N = int(rng.choice([1, 3, 8, 9, 40, 64, 100, 256, 300, 1000, 1024, 2048]))
            N = max(1, min(N, 6_000_000 // K))
            W = synth.weights(t, 9200 + 10 * case + i, N, K)
            x = synth.activations(9500 + 10 * case + i, rows, K)
            x = bf16_round(x) if bf16 else x
            b = synth.normal(9800 + 10 * case + i, 0, N).astype(np.float32) * 0.1 if rng.integers(2) else None
            act = int(rng.choice([0, 1, 2, 3]))
            hosts.append((x, W, b, act))
            xd = dev(gpu, x).to(gpu.bfloat16) if bf16 else dev(gpu, x)
            probs.append((xd, dev(gpu, W), q, None if b is None else dev(gpu, b), BACKEND_ACT[act]))
        outs = nn.quantized_dense_batch(probs, norm=norm)
        gpu.cuda.synchronize()
        for (x, W, b, act), y in zip(hosts, outs):
            xn = oracle.c_rmsnorm(x, gain, 1e-5, 0.0) if use_norm else x
            want, pre = oracle.c_qdense(t, xn, W, b, act), oracle.c_qdense(t, xn, W, b, 0)
            scale = max(float(np.max(np.abs(want))), float(np.max(np.abs(pre))))
            if not np.isfinite(scale) or scale == 0.0:
                continue
            err = float(np.max(np.abs(y.cpu().numpy().astype(np.float64) - want))) / scale
            assert err < TOL_F32, (case, ggml.name(t), rows, use_norm, bf16, W.shape, act, err)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_batches_between_decode_and_prefill_randomized(gpu, oracle, t):
    """Seeded random dense problems at 17 to 400 rows: the range in which the routes change hands (split-K kernels with one or
    several tiles of 32 rows per launch, the two-pass GEMM with and without its own split of K).  Widths that are and are not
    multiples of 4, 32 and 256, K from one to forty 256-value stretches, fp32 and bf16 activations scaled over six decades."""
    rng = np.random.default_rng(9000 + t)
    for case in range(10):
        M = int(rng.integers(17, 401))
        K = 256 * int(rng.integers(1, 41)) * (2 if t == Q6_K and rng.integers(0, 2) else 1)
        N = int(rng.choice([4 * int(rng.integers(1, 300)), 32 * int(rng.integers(1, 80)), int(rng.integers(1, 900)), 256 * int(rng.integers(1, 9))]))
        act = int(rng.choice([0, 1, 2, 3, 4]))
        W = synth.weights(t, 9100 + case, N, K)
        bias = synth.normal(9200 + case, 0, N).astype(np.float32) * 0.1 if rng.integers(0, 2) else None
        x = (synth.activations(9300 + case, M, K) * float(10.0 ** rng.uniform(-3, 3))).astype(np.float32)
        got = run_dense(gpu, t, x, W, bias, act)
        want = oracle.c_qdense(t, x, W, bias, act)
        pre = oracle.c_qdense(t, x, W, bias, 0)  # (an activation that saturates hides the contraction: judge on the larger scale)
        scale = max(float(np.max(np.abs(want))), float(np.max(np.abs(pre)))) or 1.0
        err = float(np.max(np.abs(got.astype(np.float64) - want))) / scale
        assert err < TOL_F32, (ggml.name(t), case, M, K, N, act, err)
        if case % 3 == 0:
            xb = bf16_round(x)
            got = run_dense(gpu, t, xb, W, bias, 0, bf16=True)
            assert rel_err(got, oracle.c_qdense(t, xb, W, bias, 0)) < TOL_BF16, (ggml.name(t), case, M, K, N, "bf16")


def test_shared_split_k_pass_randomized(gpu, oracle):
    """Seeded random lists of two to four Q4_K projections of one input, 6 to 99 rows, any widths that are multiples of 4
    (most not multiples of the 128-row workgroup), with and without normalisation, gain, bias; activations without tanh
    (saturated outputs measure nothing of the contraction)."""
    rng = np.random.default_rng(4242)
    q = Quantization(ggml_type=Q4_K)
    for case in range(16):
        rows, K, count = int(rng.integers(6, 100)), 256 * int(rng.integers(1, 17)), int(rng.integers(2, 5))
        Ns = [4 * int(rng.integers(1, 400)) for _ in range(count)]
        use_norm, use_gain = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        x = (synth.activations(7000 + case, rows, K) * float(10.0 ** rng.uniform(-3, 3))).astype(np.float32)
        gain = (synth.normal(7100 + case, 0, K) * 0.5 + 1.0).astype(np.float32)
        cfg = nn.RMSNorm(dev(gpu, gain) if use_gain else None, 1e-5, 0.0) if use_norm else None
        xin = oracle.c_rmsnorm(x, gain if use_gain else None, 1e-5, 0.0) if use_norm else x
        xd = dev(gpu, x)
        probs, wants = [], []
        for j, N in enumerate(Ns):
            W = synth.weights(Q4_K, 7200 + 10 * case + j, N, K)
            b = synth.normal(7300 + 10 * case + j, 0, N).astype(np.float32) * 0.1 if rng.integers(0, 2) else None
            a = int(rng.integers(0, 5))
            probs.append((xd, dev(gpu, W), q, None if b is None else dev(gpu, b), BACKEND_ACT[a]))
            wants.append(oracle.c_qdense(Q4_K, xin, W, b, a))
        outs = nn.quantized_dense_batch(probs, norm=cfg)
        gpu.cuda.synchronize()
        for y, want in zip(outs, wants):
            assert rel_err(y.cpu().numpy(), want) < TOL_F32, (case, rows, K, Ns, use_norm, use_gain)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_large_batches_with_neighbours_folded_into_the_two_passes(gpu, oracle, t):
    """From the batch sizes a plain dense call hands to the two-pass GEMM, the normalisation rides on
    the activation pass and the residual / gated product on the GEMM epilogue (fp16 operands)."""
    for i, (M, K, N, act, norm_kind, with_bias) in enumerate([(130, 1024, 132, 3, 1, True), (300, 512, 257, 1, 2, False),
                                                              (40, 768, 130, 3, 3, True), (257, 256, 64, 5, 0, True),
                                                              (256, 1024, 1000, 3, 1, True), (700, 256, 33, 2, 3, False)]):
        err = gated_case(gpu, oracle, t, M, K, N, act, norm_kind, with_bias, 820 + 10 * i + t)
        assert err < 2 * TOL_F32, ("gated", t, M, K, N, act, norm_kind, err)
    for i, (M, K, N, act, use_norm, use_res) in enumerate([(130, 1024, 132, 0, True, True), (300, 512, 257, 3, True, False),
                                                           (40, 768, 130, 0, False, True), (600, 256, 64, 2, True, True)]):
        W = synth.weights(t, 860 + i, N, K)
        x = (synth.activations(861 + i, M, K) * 3.0).astype(np.float32)
        gain = (synth.normal(862 + i, 0, K) * 0.5 + 1.0).astype(np.float32)
        bias = synth.normal(863 + i, 0, N).astype(np.float32) * 0.1
        res = synth.activations(864 + i, M, N)
        yd = dev(gpu, res)  # the residual buffer is also the output when there is a residual
        got = nn.quantized_dense(dev(gpu, x), dev(gpu, W), Quantization(ggml_type=t), dev(gpu, bias), BACKEND_ACT[act],
                                 norm=nn.RMSNorm(dev(gpu, gain), 1e-6, 0.0) if use_norm else None,
                                 residual=yd if use_res else None).cpu().numpy()
        xn = oracle.c_rmsnorm(x, gain, 1e-6, 0.0) if use_norm else x
        dense = oracle.c_qdense(t, xn, W, bias, act)
        want = dense + res if use_res else dense
        scale = max(float(np.max(np.abs(dense))), float(np.max(np.abs(oracle.c_qdense(t, xn, W, bias, 0)))))
        err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) / scale
        assert err < TOL_F32, ("block", t, M, K, N, act, use_norm, use_res, err)


def test_gated_feed_forward_full_size(gpu, oracle):
    """Llama-3-8B feed-forward front at full size (Q4_K, 4096 -> 14336 twice, RMSNorm, SiLU), checked on a
    sample of output columns against the oracle and in full against the unfused calls of this library."""
    t, K, N = Q4_K, 4096, 14336
    Wg, Wu = synth.weights(t, 800, N, K), synth.weights(t, 801, N, K)
    x = synth.activations(802, 1, K)
    gain = (synth.normal(803, 0, K) * 0.5 + 1.0).astype(np.float32)
    q = Quantization(ggml_type=t)
    xd, Wgd, Wud, gd = dev(gpu, x), dev(gpu, Wg), dev(gpu, Wu), dev(gpu, gain)
    cfg = nn.RMSNorm(gd, 1e-5, 0.0)
    got = nn.gated_feed_forward(xd, Wgd, Wud, q, Activation.SILU, norm=cfg).cpu().numpy()
    xn = nn.rms_norm(xd, cfg)
    unfused = (nn.quantized_dense(xn, Wgd, q, None, Activation.SILU) * nn.quantized_dense(xn, Wud, q)).cpu().numpy()
    scale = float(np.max(np.abs(unfused)))
    assert np.max(np.abs(got - unfused)) / scale < 1e-4
    cols = np.arange(0, N, 97)
    want = oracle.c_gated_ffn(t, x, Wg[cols], Wu[cols], None, None, 3, (gain, 1e-5, 0.0))
    assert np.max(np.abs(got[:, cols].astype(np.float64) - want)) / float(np.max(np.abs(want))) < 2 * TOL_F32


def test_gated_feed_forward_rejects_bad_arguments(gpu):
    q = Quantization(ggml_type=Q8_0)
    x = dev(gpu, np.zeros((1, 64), np.float32))
    W = dev(gpu, np.zeros((4, 68), np.uint8))
    with pytest.raises(ValueError):
        nn.gated_feed_forward(x, W, dev(gpu, np.zeros((5, 68), np.uint8)), q, Activation.SILU)
    with pytest.raises(ValueError):
        nn.gated_feed_forward(x, W, W, q, Activation.SILU, norm=nn.RMSNorm(dev(gpu, np.ones(32, np.float32))))
    with pytest.raises(Exception):
        nn.gated_feed_forward(dev(gpu, np.zeros((1, 96), np.float32)), W, W, q, Activation.SILU)
    with pytest.raises(Exception):
        nn.rms_norm(x, nn.RMSNorm(epsilon=-1.0))


def test_feed_forward_block_from_a_gguf_file(gpu, oracle, tmp_path):
    """File -> device -> kernels: the feed-forward weights of a layer stored in a GGUF container
    (llama.cpp tensor names), uploaded as Uint8 [N, bytesPerRow] and run as norm + gate/up + down."""
    from gomlx_amd import gguf
    K, F = 1024, 2816
    Wg, Wu, Wd = synth.weights(Q4_K, 900, F, K), synth.weights(Q4_K, 901, F, K), synth.weights(Q6_K, 902, K, F)
    gain = (synth.normal(903, 0, K) * 0.5 + 1.0).astype(np.float32)
    path = str(tmp_path / "layer.gguf")
    gguf.write_gguf(path, {"general.architecture": "llama", "llama.attention.layer_norm_rms_epsilon": 1e-5},
                    [("blk.0.ffn_norm.weight", 0, (K,), gain), ("blk.0.ffn_gate.weight", Q4_K, (K, F), Wg),
                     ("blk.0.ffn_up.weight", Q4_K, (K, F), Wu), ("blk.0.ffn_down.weight", Q6_K, (F, K), Wd)])
    with gguf.GGUFFile(path) as g:
        eps = float(g.metadata["llama.attention.layer_norm_rms_epsilon"])
        dg, du, dd = (g.to_device(f"blk.0.ffn_{n}.weight") for n in ("gate", "up", "down"))
        dn = g.to_device("blk.0.ffn_norm.weight")
        types = {n: g.tensors[f"blk.0.ffn_{n}.weight"].ggml_type for n in ("gate", "up", "down")}
    assert dg.dtype == gpu.uint8 and tuple(dg.shape) == (F, ggml.row_bytes(Q4_K, K)) and dn.dtype == gpu.float32
    assert types == {"gate": Q4_K, "up": Q4_K, "down": Q6_K}
    x = synth.activations(904, 2, K)
    ff = nn.gated_feed_forward(dev(gpu, x), dg, du, Quantization(ggml_type=types["gate"]), Activation.SILU, norm=nn.RMSNorm(dn, eps))
    y = nn.quantized_dense(ff, dd, Quantization(ggml_type=types["down"])).cpu().numpy()
    ff_want = oracle.c_gated_ffn(Q4_K, x, Wg, Wu, None, None, 3, (gain, eps, 0.0))
    want = oracle.c_qdense(Q6_K, ff_want, Wd)
    assert rel_err(ff.cpu().numpy(), ff_want) < 2 * TOL_F32
    assert rel_err(y, want) < 2 * TOL_F32


# ------------------------------------------------------------------------------ benchmark configurations, full size

def test_config0_q8_0_gemv_4096(gpu, oracle):
    W = synth.weights(Q8_0, 1000, 4096, 4096)
    x = synth.activations(1000, 1, 4096)
    assert rel_err(run_dense(gpu, Q8_0, x, W), oracle.c_qdense(Q8_0, x, W)) < TOL_F32


def test_config1_q4_0_gemv_14336(gpu, oracle):
    W = synth.weights(Q4_0, 1001, 14336, 4096)
    x = synth.activations(1001, 1, 4096)
    assert rel_err(run_dense(gpu, Q4_0, x, W), oracle.c_qdense(Q4_0, x, W)) < TOL_F32


def test_config2_q4_k_batch32(gpu, oracle):
    W = synth.weights(Q4_K, 1002, 4096, 14336)
    x = synth.activations(1002, 32, 14336)
    assert rel_err(run_dense(gpu, Q4_K, x, W), oracle.c_qdense(Q4_K, x, W)) < TOL_F32


@pytest.mark.parametrize("M,K,N", [(32, 14336, 4096), (9, 4096, 1024), (40, 2048, 896)])
def test_q4_k_split_k_stages_missing_activation_records_itself(gpu, oracle, M, K, N, monkeypatch):
    """The Q4_K split-K kernel's workgroups share the staging of the activations through memory and flag words.  With the
    bound on the wait for those flags at zero every wait runs out at once (forced from the host; the kernel exits normally)
    and each workgroup stages what it misses itself: the results must be the same bits as with the default bound, and within
    the bound of the oracle.  bf16 rows as well (widened exactly)."""
    torch = gpu
    W = synth.weights(Q4_K, 1302, N, K)
    x = synth.activations(1303, M, K)
    want = oracle.c_qdense(Q4_K, x, W)
    monkeypatch.setenv("GOMLX_HIPQ_COOP", "1")  # (the route is not the default: it measured slower than the three launches)
    monkeypatch.delenv("GOMLX_HIPQ_COOP_SPIN_TICKS", raising=False)
    ref = run_dense(torch, Q4_K, x, W)
    assert rel_err(ref, want) < TOL_F32
    monkeypatch.setenv("GOMLX_HIPQ_COOP_SPIN_TICKS", "0")
    for _ in range(2):
        assert np.array_equal(run_dense(torch, Q4_K, x, W).view(np.uint32), ref.view(np.uint32))
    xb = bf16_round(x)
    got_b = run_dense(torch, Q4_K, xb, W, bf16=True)
    monkeypatch.delenv("GOMLX_HIPQ_COOP_SPIN_TICKS")
    assert np.array_equal(run_dense(torch, Q4_K, xb, W, bf16=True).view(np.uint32), got_b.view(np.uint32))
    assert rel_err(got_b, oracle.c_qdense(Q4_K, xb, W)) < TOL_F32
    # the three-launch route (separate pre-pass) agrees to rounding: its activations carry one scale per slice, not per super-block
    monkeypatch.delenv("GOMLX_HIPQ_COOP")
    assert rel_err(run_dense(torch, Q4_K, x, W), want) < TOL_F32


def test_config3_q8_0_prefill_bf16(gpu, oracle):
    W = synth.weights(Q8_0, 1000, 4096, 4096)
    x = bf16_round(synth.activations(1003, 2048, 4096))
    got = run_dense(gpu, Q8_0, x, W, bf16=True)
    rows = np.array([0, 1, 31, 32, 127, 128, 1000, 2047])
    want = oracle.c_qdense(Q8_0, x[rows], W)
    assert got.shape == (2048, 4096)
    assert rel_err(got[rows], want) < TOL_BF16
    # size-independent property on the whole output: duplicated activation rows give identical rows
    x2 = x.copy()
    x2[1024:] = x2[:1024]
    got2 = run_dense(gpu, Q8_0, x2, W, bf16=True)
    assert np.array_equal(got2[:1024], got2[1024:])
    assert np.array_equal(got2[:1024], got[:1024])


def test_config4_llama_layer_projections(gpu, oracle):
    shapes = [(4096, 4096), (4096, 1024), (4096, 1024), (4096, 4096), (4096, 14336), (4096, 14336), (14336, 4096)]
    for i, (K, N) in enumerate(shapes):
        W = synth.weights(Q4_K, 1004 + i, N, K)
        x = synth.activations(1104 + i, 1, K)
        assert rel_err(run_dense(gpu, Q4_K, x, W), oracle.c_qdense(Q4_K, x, W)) < TOL_F32, (K, N)


C4_SHAPES = [(4096, 4096), (4096, 1024), (4096, 1024), (4096, 4096), (4096, 14336), (4096, 14336), (14336, 4096)]


@pytest.mark.parametrize("rows", [1, 2, 3])
def test_config4_seven_projections_as_one_batched_submission(gpu, oracle, rows):
    """Configuration 4 the way the benchmark times it: the seven full-size Q4_K matrices handed over in ONE
    gq_qdense_f32_batch (one launch of the batched decode GEMV, whose plan deals every matrix's rows over a common grid),
    against the oracle and, bit for bit, against seven separate calls.  Two and three rows per problem as well."""
    torch = gpu
    q = Quantization(ggml_type=Q4_K)
    hosts, probs = [], []
    for i, (K, N) in enumerate(C4_SHAPES):
        W = synth.weights(Q4_K, 1004 + i, N, K)
        x = synth.activations(1104 + i, rows, K)
        hosts.append((x, W))
        probs.append((dev(torch, x), dev(torch, W), q, None, Activation.NONE))
    outs = nn.quantized_dense_batch(probs)
    torch.cuda.synchronize()
    for (x, W), p, y in zip(hosts, probs, outs):
        assert rel_err(y.cpu().numpy(), oracle.c_qdense(Q4_K, x, W)) < TOL_F32, (rows, W.shape)
        assert torch.equal(nn.quantized_dense(p[0], p[1], q), y), (rows, W.shape)


@pytest.mark.parametrize("rows", [1, 2])
def test_decoder_layer_sequence_full_size(gpu, oracle, rows):
    """Configuration 4's matrices in the order and with the dependencies of a decoder layer, at full size, as four calls:
    q / k / v behind one RMSNorm (one submission), o + residual, RMSNorm + act(gate) * up, down + residual in place.
    Every call is judged against the oracle on the inputs that call received (so each keeps the 1e-3 bound of a single
    contraction, 2e-3 for the product of two), and the end of the chain against the oracle's own chain."""
    import ctypes
    from gomlx_amd import _lib
    torch = gpu
    L = _lib.lib()
    t = Q4_K
    Ws = [synth.weights(t, 1004 + i, N, K) for i, (K, N) in enumerate(C4_SHAPES)]
    Wq, Wk, Wv, Wo, Wg, Wu, Wd = (dev(torch, W) for W in Ws)
    H, KV, F = 4096, 1024, 14336
    x0 = synth.activations(1104, rows, H)
    # The rows of these synthetic weights all have the same positive mean, so every output of a projection carries the sum
    # of its input: an attention output with a positive mean keeps the gates on the rising side of SiLU (with a negative
    # one act(gate) * up collapses to ~1e-5 and the last call would only test the residual), and a small gain keeps the
    # down projection at the magnitude of the residual it is added to, so that both show in the result.
    attn0 = synth.activations(1107, rows, H) + np.float32(0.25)
    gain = ((synth.normal(1200, 0, H) * 0.5 + 1.0) * 3e-4).astype(np.float32)
    eps = 1e-5
    x, attn, gd = dev(torch, x0), dev(torch, attn0), dev(torch, gain)
    q, k, v = (torch.full((rows, n), float("nan"), device="cuda") for n in (H, KV, KV))
    h, ff = torch.full((rows, H), float("nan"), device="cuda"), torch.full((rows, F), float("nan"), device="cuda")
    norm = _lib.RmsNormDesc(gd.data_ptr(), eps, 0.0)
    sp = torch.cuda.current_stream().cuda_stream
    d = (_lib.DenseDesc * 3)()
    for dd, (W, y, n) in zip(d, ((Wq, q, H), (Wk, k, KV), (Wv, v, KV))):
        dd.type, dd.act, dd.dX, dd.M, dd.K, dd.dW, dd.N, dd.dBias, dd.dY = t, 0, x.data_ptr(), rows, H, W.data_ptr(), n, None, y.data_ptr()
    _lib.check(L.gq_qdense_norm_f32_batch(3, d, ctypes.byref(norm), sp))
    _lib.check(L.gq_qdense_block_f32(t, attn.data_ptr(), rows, H, None, Wo.data_ptr(), H, None, 0, x.data_ptr(), h.data_ptr(), sp))
    _lib.check(L.gq_qdense_gated_f32(t, h.data_ptr(), rows, H, ctypes.byref(norm), Wg.data_ptr(), None, Wu.data_ptr(), None, F, 3,
                                     ff.data_ptr(), sp))
    torch.cuda.synchronize()
    h_mid = h.cpu().numpy()
    _lib.check(L.gq_qdense_block_f32(t, ff.data_ptr(), rows, F, None, Wd.data_ptr(), H, None, 0, h.data_ptr(), h.data_ptr(), sp))
    torch.cuda.synchronize()

    def close(got, dense, res, tol, what):  # the bound is on the contraction; a residual only shifts both sides
        want = dense if res is None else dense + res
        err = float(np.max(np.abs(got.astype(np.float64) - want)))
        rel_err(got, want)  # (records the margins)
        # (the addition of the residual is one more fp32 rounding, of the sum)
        assert err < tol * float(np.max(np.abs(dense))) + 2.0 ** -23 * float(np.max(np.abs(want))), (what, rows, err)

    xn = oracle.c_rmsnorm(x0, gain, eps, 0.0)
    for got, W, what in ((q, Ws[0], "q"), (k, Ws[1], "k"), (v, Ws[2], "v")):
        close(got.cpu().numpy(), oracle.c_qdense(t, xn, W), None, TOL_F32, what)
    close(h_mid, oracle.c_qdense(t, attn0, Ws[3]), x0.astype(np.float64), TOL_F32, "o + residual")
    ff_got = ff.cpu().numpy()
    hn = oracle.c_rmsnorm(h_mid, gain, eps, 0.0)
    g_pre, u_pre = oracle.c_qdense(t, hn, Ws[4]), oracle.c_qdense(t, hn, Ws[5])
    ff_want = oracle.c_gated_ffn(t, h_mid, Ws[4], Ws[5], None, None, 3, (gain, eps, 0.0))
    assert np.max(np.abs(ff_got.astype(np.float64) - ff_want)) / (float(np.max(np.abs(g_pre))) * float(np.max(np.abs(u_pre)))) < 2 * TOL_F32
    out = h.cpu().numpy()
    close(out, oracle.c_qdense(t, ff_got, Ws[6]), h_mid.astype(np.float64), TOL_F32, "down + residual")
    # the oracle's own chain from the layer's inputs (the errors of three contractions in a row add up)
    h_o = (oracle.c_qdense(t, attn0, Ws[3]) + x0).astype(np.float32)
    ff_o = oracle.c_gated_ffn(t, h_o, Ws[4], Ws[5], None, None, 3, (gain, eps, 0.0)).astype(np.float32)
    dense_o = oracle.c_qdense(t, ff_o, Ws[6])
    assert float(np.max(np.abs(ff_got))) > 0.05 and float(np.max(np.abs(dense_o))) > 0.1 * float(np.max(np.abs(h_o)))  # (not degenerate)
    assert float(np.max(np.abs(out.astype(np.float64) - (dense_o + h_o)))) / float(np.max(np.abs(dense_o))) < 4 * TOL_F32


def test_batched_submission_equals_separate_calls(gpu, oracle):
    """gq_qdense_f32_batch: the seven projections of a decoder layer (scaled down), mixed with a
    batch-5 problem and another format, against one call each and against the oracle."""
    torch = gpu
    shapes = [(1024, 1024), (1024, 256), (1024, 256), (1024, 1024), (1024, 3584), (1024, 3584), (3584, 1024)]
    probs, hosts = [], []
    for i, (K, N) in enumerate(shapes):
        W = synth.weights(Q4_K, 170 + i, N, K)
        x = synth.activations(180 + i, 1, K)
        b = synth.normal(190 + i, 0, N).astype(np.float32) * 0.1 if i % 2 else None
        act = Activation.SILU if i == 4 else Activation.NONE
        hosts.append((Q4_K, x, W, b, act))
    hosts.append((Q4_K, synth.activations(200, 5, 512), synth.weights(Q4_K, 201, 64, 512), None, Activation.NONE))
    hosts.append((Q8_0, synth.activations(202, 1, 2048), synth.weights(Q8_0, 203, 300, 2048), None, Activation.RELU))
    hosts.append((Q8_0, synth.activations(204, 1, 2048), synth.weights(Q8_0, 205, 77, 2048), None, Activation.NONE))
    # two problems whose K is an odd multiple of 256 (half tail slice) share a launch too
    hosts.append((Q4_0, synth.activations(212, 1, 1280), synth.weights(Q4_0, 213, 200, 1280), None, Activation.NONE))
    hosts.append((Q4_0, synth.activations(214, 1, 4864), synth.weights(Q4_0, 215, 64, 4864), None, Activation.NONE))
    # a run of Q6_K problems (K-sliced kernels only), then one whose K has no K-sliced plan
    hosts.append((Q6_K, synth.activations(206, 1, 1024), synth.weights(Q6_K, 207, 256, 1024), None, Activation.NONE))
    hosts.append((Q6_K, synth.activations(208, 1, 1024), synth.weights(Q6_K, 209, 520, 1024), None, Activation.GELU))
    hosts.append((Q8_0, synth.activations(210, 1, 96), synth.weights(Q8_0, 211, 100, 96), None, Activation.NONE))
    for t, x, W, b, act in hosts:
        probs.append((dev(torch, x), dev(torch, W), Quantization(ggml_type=t), None if b is None else dev(torch, b), act))
    outs = nn.quantized_dense_batch(probs)
    torch.cuda.synchronize()
    for (t, x, W, b, act), p, y in zip(hosts, probs, outs):
        single = nn.quantized_dense(p[0], p[1], p[2], p[3], act)
        assert torch.equal(single, y)
        want = oracle.c_qdense(t, x, W, b, act.to_backend())
        assert rel_err(y.cpu().numpy(), want) < TOL_F32


# ------------------------------------------------------------------------------ gather

@pytest.mark.parametrize("t", ALL_TYPES)
def test_gather_random_rows_bit_exact(gpu, oracle, t):
    vocab, K = 1000, 512
    table = synth.weights(t, 110 + t, vocab, K)
    idx = synth.randint(111, t, 2 * 77, 0, vocab - 1).astype(np.int32).reshape(2, 77, 1)
    out = nn.quantized_gather(dev(gpu, table), dev(gpu, idx), Quantization(ggml_type=t)).cpu().numpy()
    want = oracle.c_embedding_lookup(t, table, K, idx)
    assert out.shape == (2, 77, K)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


def test_gather_out_of_range_index_raises(gpu):
    table = synth.weights(Q8_0, 120, 10, 64)
    for bad in (10, -1):
        with pytest.raises(IndexError):
            nn.quantized_gather(dev(gpu, table), dev(gpu, np.array([[3], [bad]], np.int32)), Quantization(ggml_type=Q8_0))


# ------------------------------------------------------------------------------ recorded replays and timing hooks

def test_recorded_chain_replays_match_eager(gpu, oracle):
    """Seven projections recorded once (HIP graph) and replayed; every replay must equal the
    eager result, with eager work and synchronisations in between."""
    from gomlx_amd import _lib
    torch = gpu
    L = _lib.lib()
    shapes = [(1024, 512), (1024, 256), (1024, 256), (1024, 512), (1024, 1536), (1024, 1536), (1536, 1024)]
    Ws = [dev(torch, synth.weights(Q4_K, 130 + i, N, K)) for i, (K, N) in enumerate(shapes)]
    xs = [dev(torch, synth.activations(140 + i, 1, K)) for i, (K, N) in enumerate(shapes)]
    ys = [torch.zeros(1, N, device="cuda") for (K, N) in shapes]
    eager = [nn.quantized_dense(x, W, Quantization(ggml_type=Q4_K)).clone() for x, W in zip(xs, Ws)]
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    sp = stream.cuda_stream
    _lib.check(L.gq_graph_begin(sp))
    for (K, N), x, W, y in zip(shapes, xs, Ws, ys):
        _lib.check(L.gq_qdense_f32(Q4_K, x.data_ptr(), 1, K, W.data_ptr(), N, None, 0, y.data_ptr(), sp))
    import ctypes
    g = ctypes.c_void_p()
    _lib.check(L.gq_graph_end(sp, ctypes.byref(g)))
    for rep in range(4):
        for y in ys:
            y.fill_(float("nan"))
        torch.cuda.synchronize()
        _lib.check(L.gq_graph_launch(g, sp))
        _lib.check(L.gq_sync(sp))
        for y, e in zip(ys, eager):
            assert torch.equal(y, e), rep
        # eager work between replays
        again = nn.quantized_dense(xs[0], Ws[0], Quantization(ggml_type=Q4_K))
        torch.cuda.synchronize()
        assert torch.equal(again, eager[0])
    _lib.check(L.gq_graph_destroy(g))


def test_recording_needs_the_stream_workspace_to_exist(gpu, oracle):
    """Paths with a workspace (here the two-pass GEMM) refuse to allocate inside a recording: the
    call reports an error, the recording stays usable, and after one eager call on the stream the
    same recording works and replays exactly."""
    import ctypes
    from gomlx_amd import _lib
    torch = gpu
    L = _lib.lib()
    M, K, N = 600, 256, 128
    W = dev(torch, synth.weights(Q4_0, 150, N, K))
    x = dev(torch, synth.activations(151, M, K))
    x1 = dev(torch, synth.activations(152, 1, K))
    y = torch.zeros(M, N, device="cuda")
    y1 = torch.zeros(1, N, device="cuda")
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()  # a fresh stream: no workspace yet
    sp = stream.cuda_stream
    dense = lambda xx, rows, yy: L.gq_qdense_f32(Q4_0, xx.data_ptr(), rows, K, W.data_ptr(), N, None, 0, yy.data_ptr(), sp)
    _lib.check(L.gq_graph_begin(sp))
    _lib.check(dense(x1, 1, y1))  # a path without workspace records fine
    rc = dense(x, M, y)
    assert rc == _lib.ERR_INVALID
    assert b"workspace" in L.gq_last_error()
    g = ctypes.c_void_p()
    _lib.check(L.gq_graph_end(sp, ctypes.byref(g)))
    _lib.check(L.gq_graph_destroy(g))
    _lib.check(dense(x, M, y))  # eager: creates the stream's workspace
    _lib.check(L.gq_sync(sp))
    eager = y.clone()
    assert rel_err(eager.cpu().numpy(), oracle.c_qdense(Q4_0, x.cpu().numpy(), W.cpu().numpy())) < TOL_F32
    _lib.check(L.gq_graph_begin(sp))
    _lib.check(dense(x, M, y))
    _lib.check(L.gq_graph_end(sp, ctypes.byref(g)))
    for rep in range(3):
        y.fill_(float("nan"))
        torch.cuda.synchronize()
        _lib.check(L.gq_graph_launch(g, sp))
        _lib.check(L.gq_sync(sp))
        assert torch.equal(y, eager), rep
    _lib.check(L.gq_graph_destroy(g))


def test_kernel_timing_hook_counts_launches(gpu):
    from gomlx_amd import _lib
    import ctypes
    L = _lib.lib()
    W = dev(gpu, synth.weights(Q8_0, 150, 512, 1024))
    x = dev(gpu, synth.activations(151, 1, 1024))
    ref = nn.quantized_dense(x, W, Quantization(ggml_type=Q8_0))
    _lib.check(L.gq_profile_begin())
    outs = [nn.quantized_dense(x, W, Quantization(ggml_type=Q8_0)) for _ in range(5)]
    n, us = ctypes.c_int(0), ctypes.c_double(0.0)
    _lib.check(L.gq_profile_end(ctypes.byref(n), ctypes.byref(us)))
    assert n.value == 5 and 0.0 < us.value < 5e4
    for o in outs:
        assert gpu.equal(o, ref)


# ------------------------------------------------------------------------------ operator-level error behaviour

def test_operator_rejects_bad_arguments(gpu):
    from gomlx_amd import _lib
    W = dev(gpu, synth.weights(Q8_0, 160, 8, 64))
    x = gpu.zeros((1, 64), device="cuda")
    q = Quantization(ggml_type=Q8_0)
    with pytest.raises(_lib.HipqError):            # x features != K (ml/ggml/dense.go:38-41)
        nn.quantized_dense(gpu.zeros((1, 96), device="cuda"), W, q)
    with pytest.raises(_lib.HipqError):            # bias length
        nn.quantized_dense(x, W, q, gpu.zeros(7, device="cuda"))
    with pytest.raises(ValueError):                # more than one activation (quantized_dense.go:35-38)
        nn.quantized_dense(x, W, q, None, Activation.RELU, Activation.TANH)
    with pytest.raises(_lib.NotImplementedByBackend):
        nn.quantized_dense(x, W, Quantization(scheme=nn.QuantizationScheme.NF4))
    with pytest.raises(_lib.NotImplementedByBackend):
        nn.quantized_dense(x.to(gpu.float16), W, q)
    with pytest.raises(ValueError):                # CPU tensors: there is no CPU path
        nn.quantized_dense(x.cpu(), W, q)
    # activations without a backend enum are dropped on the fused route (activation.go:72-73)
    y0 = nn.quantized_dense(x + 1.0, W, q)
    y1 = nn.quantized_dense(x + 1.0, W, q, None, Activation.SIGMOID)
    assert gpu.equal(y0, y1)


@pytest.mark.parametrize("rows", [1, 3, 24, 100, 300])
def test_decoder_layer_calls_replay_as_a_graph(gpu, rows):
    """The calls of a decoder layer (q/k/v behind a norm, o + residual, norm + gate/up product, down +
    residual in place) recorded once and replayed four times, with eager work between the replays:
    every replay must reproduce the eager results exactly.  Batch sizes of all three kernel
    families (100 rows: the split-K kernel that walks four tiles of 32 rows); one eager pass first creates the workspaces the larger ones need."""
    import ctypes
    from gomlx_amd import _lib
    torch = gpu
    L = _lib.lib()
    t, H, KV, F = Q4_K, 512, 256, 1024
    mk = lambda seed, n, k: dev(torch, synth.weights(t, seed, n, k))
    Wq, Wk, Wv, Wo, Wg, Wu, Wd = mk(1, H, H), mk(2, KV, H), mk(3, KV, H), mk(4, H, H), mk(5, F, H), mk(6, F, H), mk(7, H, F)
    x0 = dev(torch, synth.activations(8, rows, H))
    attn = dev(torch, synth.activations(9, rows, H))
    # (a small gain keeps the gated product of these synthetic weights inside the fp16 range that the
    # activations of the MFMA paths are rounded to)
    g1 = dev(torch, ((synth.normal(10, 0, H) * 0.5 + 1.0) * 0.02).astype(np.float32))
    q, k, v = (torch.zeros(rows, n, device="cuda") for n in (H, KV, KV))
    h, ff, x = torch.zeros(rows, H, device="cuda"), torch.zeros(rows, F, device="cuda"), torch.zeros(rows, H, device="cuda")
    norm = _lib.RmsNormDesc(g1.data_ptr(), 1e-5, 0.0)
    stream = torch.cuda.Stream()
    sp = stream.cuda_stream

    def layer():
        d = (_lib.DenseDesc * 3)()
        for dd, (W, y, n) in zip(d, ((Wq, q, H), (Wk, k, KV), (Wv, v, KV))):
            dd.type, dd.act, dd.dX, dd.M, dd.K, dd.dW, dd.N, dd.dBias, dd.dY = t, 0, x.data_ptr(), rows, H, W.data_ptr(), n, None, y.data_ptr()
        _lib.check(L.gq_qdense_norm_f32_batch(3, d, ctypes.byref(norm), sp))
        _lib.check(L.gq_qdense_block_f32(t, attn.data_ptr(), rows, H, None, Wo.data_ptr(), H, None, 0, x.data_ptr(), h.data_ptr(), sp))
        _lib.check(L.gq_qdense_gated_f32(t, h.data_ptr(), rows, H, ctypes.byref(norm), Wg.data_ptr(), None, Wu.data_ptr(), None, F, 3,
                                         ff.data_ptr(), sp))
        _lib.check(L.gq_qdense_block_f32(t, ff.data_ptr(), rows, F, None, Wd.data_ptr(), H, None, 0, h.data_ptr(), h.data_ptr(), sp))

    def reset():
        x.copy_(x0)
        for b in (q, k, v, h, ff):
            b.fill_(float("nan"))
        torch.cuda.synchronize()

    reset()
    layer()
    _lib.check(L.gq_sync(sp))
    eager = [b.clone() for b in (q, k, v, h, ff)]
    assert all(bool(torch.isfinite(b).all()) for b in eager)
    _lib.check(L.gq_graph_begin(sp))
    layer()
    g = ctypes.c_void_p()
    _lib.check(L.gq_graph_end(sp, ctypes.byref(g)))
    for rep in range(4):
        reset()
        _lib.check(L.gq_graph_launch(g, sp))
        _lib.check(L.gq_sync(sp))
        for got, want in zip((q, k, v, h, ff), eager):
            assert torch.equal(got, want), rep
        (x0 * 2.0).sum().item()  # unrelated eager work and a synchronisation between replays
    _lib.check(L.gq_graph_destroy(g))

