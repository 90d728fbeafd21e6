/*
 * CPU oracle for GoMLX's quantized Dense path.  TEST INFRASTRUCTURE ONLY - see
 * ggml_oracle.h for the rules and the pinning status of each function.
 *
 * Build with -ffp-contract=off: every fp32 multiply / subtract below must round
 * on its own, exactly like the separate Mul / Sub graph nodes of the reference.
 */
#include "ggml_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- fp16 ------------------------------------------------------------- */

float gqo_fp16_to_fp32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign; /* +-0 */
        } else {     /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while ((man & 0x400u) == 0);
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13); /* inf / nan (payload kept) */
    } else {
        bits = sign | ((exp + (127 - 15)) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
}

static inline uint16_t load_u16le(const uint8_t *p) {
    return (uint16_t)(p[0] | ((uint16_t)p[1] << 8));
}

/* ---- block geometry --------------------------------------------------- */

int gqo_bytes_per_block(int type) {
    switch (type) {
    case GQO_Q4_0: return 18;
    case GQO_Q8_0: return 34;
    case GQO_Q4_K: return 144;
    case GQO_Q6_K: return 210;
    case GQO_IQ4_NL: return 18;
    default: return 0;
    }
}

int gqo_values_per_block(int type) {
    switch (type) {
    case GQO_Q4_0: case GQO_Q8_0: case GQO_IQ4_NL: return 32;
    case GQO_Q4_K: case GQO_Q6_K: return 256;
    default: return 0;
    }
}

size_t gqo_row_bytes(int type, int64_t K) {
    const int vpb = gqo_values_per_block(type);
    if (vpb == 0 || K <= 0 || K % vpb != 0) return 0;
    return (size_t)(K / vpb) * (size_t)gqo_bytes_per_block(type);
}

/* ---- per-block dequantisation ----------------------------------------- */

/* dequantQ8_0, ml/ggml/dequant.go:58-78: bytes 0-1 fp16 d, bytes 2-33 int8 q;
 * w[i] = f32(q[i]) * f32(d). */
static void dequant_block_q8_0(const uint8_t *b, float *out) {
    const float d = gqo_fp16_to_fp32(load_u16le(b));
    for (int i = 0; i < 32; i++) out[i] = (float)(int8_t)b[2 + i] * d;
}

/* extractNibbleBlock + dequantQ4_0, ml/ggml/dequant.go:83-115: low nibbles of the
 * 16 packed bytes are values 0..15, high nibbles values 16..31;
 * w[i] = (f32(nibble) - 8.0f) * f32(d). */
static void dequant_block_q4_0(const uint8_t *b, float *out) {
    const float d = gqo_fp16_to_fp32(load_u16le(b));
    for (int j = 0; j < 16; j++) {
        const uint8_t v = b[2 + j];
        out[j] = ((float)(v & 0x0F) - 8.0f) * d;
        out[j + 16] = ((float)(v >> 4) - 8.0f) * d;
    }
}

/* Public GGML non-linear 4-bit table (compute.IQ4NLLookupTable, used at
 * ml/ggml/dequant.go:130; entries 8 and 9 are pinned by
 * ml/nn/quantized_dense_test.go:409-410). */
static const float kIQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10,
                                 1, 13, 25, 38, 53, 69, 89, 113};

/* dequantIQ4NL, ml/ggml/dequant.go:121-136: Q4_0 layout, w[i] = LUT[nibble] * f32(d). */
static void dequant_block_iq4_nl(const uint8_t *b, float *out) {
    const float d = gqo_fp16_to_fp32(load_u16le(b));
    for (int j = 0; j < 16; j++) {
        const uint8_t v = b[2 + j];
        out[j] = kIQ4NL[v & 0x0F] * d;
        out[j + 16] = kIQ4NL[v >> 4] * d;
    }
}

/* Q4_K super-block (public GGML block_q4_K; reached from
 * ml/nn/quantized_dense.go:56, arithmetic in the un-vendored
 * github.com/gomlx/compute v0.1.2 - PARITY UNPINNED):
 *   bytes 0-1 fp16 d, 2-3 fp16 dmin, 4-15 packed 6-bit (scale,min) x 8, 16-143 codes.
 *   sub-block j<4 : sc = s[j] & 63,                      m = s[j+4] & 63
 *   sub-block j>=4: sc = (s[j+4] & 15) | (s[j-4] >> 6) << 4, m = (s[j+4] >> 4) | (s[j] >> 6) << 4
 *   codes: group g of 64 values uses bytes qs[32g .. 32g+31]; low nibbles are values
 *   64g+0..31 (sub-block 2g), high nibbles values 64g+32..63 (sub-block 2g+1).
 *   w = (f32(d) * sc) * q - (f32(dmin) * m), each operation rounded to fp32. */
static void q4k_scale_min(const uint8_t *s, int j, int *sc, int *m) {
    if (j < 4) {
        *sc = s[j] & 63;
        *m = s[j + 4] & 63;
    } else {
        *sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4);
        *m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

static void dequant_block_q4_k(const uint8_t *b, float *out) {
    const float d = gqo_fp16_to_fp32(load_u16le(b));
    const float dmin = gqo_fp16_to_fp32(load_u16le(b + 2));
    const uint8_t *s = b + 4;
    const uint8_t *qs = b + 16;
    for (int g = 0; g < 4; g++) {
        int sc, m;
        q4k_scale_min(s, 2 * g, &sc, &m);
        const float d1 = d * (float)sc, m1 = dmin * (float)m;
        q4k_scale_min(s, 2 * g + 1, &sc, &m);
        const float d2 = d * (float)sc, m2 = dmin * (float)m;
        for (int l = 0; l < 32; l++) {
            const uint8_t v = qs[32 * g + l];
            out[64 * g + l] = d1 * (float)(v & 0x0F) - m1;
            out[64 * g + 32 + l] = d2 * (float)(v >> 4) - m2;
        }
    }
}

/* Q6_K super-block (public GGML block_q6_K; listed by the reference among the GGMLQuantType values,
 * docs/CHANGELOG.md:251-252, and reached from ml/nn/quantized_dense.go:56; arithmetic in the
 * un-vendored github.com/gomlx/compute v0.1.2 - PARITY UNPINNED):
 *   bytes 0-127 ql (low 4 bits), 128-191 qh (high 2 bits), 192-207 int8 scales x 16, 208-209 fp16 d.
 *   For each half h of 128 values and l = 0..31:
 *     value 128h + l      : ql[64h + l] & 15      | ((qh[32h + l] >> 0) & 3) << 4, scale 8h + l/16
 *     value 128h + 32 + l : ql[64h + 32 + l] & 15 | ((qh[32h + l] >> 2) & 3) << 4, scale 8h + 2 + l/16
 *     value 128h + 64 + l : ql[64h + l] >> 4      | ((qh[32h + l] >> 4) & 3) << 4, scale 8h + 4 + l/16
 *     value 128h + 96 + l : ql[64h + 32 + l] >> 4 | ((qh[32h + l] >> 6) & 3) << 4, scale 8h + 6 + l/16
 *   w = (f32(d) * scale) * (q - 32).  The exact product has at most 11 + 7 + 6 = 24 significant
 *   bits, so every evaluation order gives the same fp32 value (denormal results aside). */
static void dequant_block_q6_k(const uint8_t *b, float *out) {
    const uint8_t *ql = b, *qh = b + 128;
    const int8_t *sc = (const int8_t *)(b + 192);
    const float d = gqo_fp16_to_fp32(load_u16le(b + 208));
    for (int h = 0; h < 2; h++) {
        for (int l = 0; l < 32; l++) {
            const int is = l / 16;
            const int q1 = (int)((ql[64 * h + l] & 0x0F) | (((qh[32 * h + l] >> 0) & 3) << 4)) - 32;
            const int q2 = (int)((ql[64 * h + 32 + l] & 0x0F) | (((qh[32 * h + l] >> 2) & 3) << 4)) - 32;
            const int q3 = (int)((ql[64 * h + l] >> 4) | (((qh[32 * h + l] >> 4) & 3) << 4)) - 32;
            const int q4 = (int)((ql[64 * h + 32 + l] >> 4) | (((qh[32 * h + l] >> 6) & 3) << 4)) - 32;
            out[128 * h + l] = (d * (float)sc[8 * h + is]) * (float)q1;
            out[128 * h + 32 + l] = (d * (float)sc[8 * h + 2 + is]) * (float)q2;
            out[128 * h + 64 + l] = (d * (float)sc[8 * h + 4 + is]) * (float)q3;
            out[128 * h + 96 + l] = (d * (float)sc[8 * h + 6 + is]) * (float)q4;
        }
    }
}

typedef void (*block_fn)(const uint8_t *, float *);

static block_fn block_dequantizer(int type) {
    switch (type) {
    case GQO_Q8_0: return dequant_block_q8_0;
    case GQO_Q4_0: return dequant_block_q4_0;
    case GQO_Q4_K: return dequant_block_q4_k;
    case GQO_Q6_K: return dequant_block_q6_k;
    case GQO_IQ4_NL: return dequant_block_iq4_nl;
    default: return NULL;
    }
}

static void dequant_row(block_fn fn, int bpb, int vpb, const uint8_t *row, int64_t K, float *out) {
    const int64_t nb = K / vpb;
    for (int64_t b = 0; b < nb; b++) fn(row + b * bpb, out + b * vpb);
}

int gqo_dequantize(int type, const uint8_t *W, int64_t N, int64_t K, float *out) {
    block_fn fn = block_dequantizer(type);
    const size_t rb = gqo_row_bytes(type, K);
    if (!fn || rb == 0) return -1;
    const int bpb = gqo_bytes_per_block(type), vpb = gqo_values_per_block(type);
    for (int64_t n = 0; n < N; n++) dequant_row(fn, bpb, vpb, W + (size_t)n * rb, K, out + (size_t)n * K);
    return 0;
}

/* ---- epilogue --------------------------------------------------------- */

/* The fused op receives compute.ActivationType, to which both TypeGelu and
 * TypeGeluApprox map (activation.go:62-63); the exact erf form is used here, the one
 * activation.Gelu requests from the backend (BackendFusedGelu(x, true),
 * activation.go:275-276).  Evaluated in double and rounded once. */
float gqo_activation(int act, float v) {
    const double x = (double)v;
    switch (act) {
    case GQO_ACT_NONE: return v;
    case GQO_ACT_RELU: return v > 0.0f ? v : 0.0f;                  /* activation.go:161 */
    case GQO_ACT_SILU: return (float)(x / (1.0 + exp(-x)));         /* activation.go:195 */
    case GQO_ACT_HARDSWISH: {                                       /* activation.go:222-243 */
        double c = x / 6.0 + 0.5;
        c = c < 0.0 ? 0.0 : (c > 1.0 ? 1.0 : c);
        return (float)(x * c);
    }
    case GQO_ACT_TANH: return (float)tanh(x);
    case GQO_ACT_GELU: return (float)(x * 0.5 * (1.0 + erf(x / sqrt(2.0)))); /* activation.go:274-286 */
    default: return NAN;
    }
}

/* ---- dense ------------------------------------------------------------ */

int gqo_qdense(int type, const float *x, int64_t M, int64_t K, const uint8_t *W,
               int64_t N, const float *bias, int act, float *y) {
    block_fn fn = block_dequantizer(type);
    const size_t rb = gqo_row_bytes(type, K);
    if (!fn || rb == 0 || act < GQO_ACT_NONE || act > GQO_ACT_TANH) return -1;
    const int bpb = gqo_bytes_per_block(type), vpb = gqo_values_per_block(type);
    float *wrow = (float *)malloc((size_t)K * sizeof(float));
    if (!wrow) return -3;
    for (int64_t n = 0; n < N; n++) {
        dequant_row(fn, bpb, vpb, W + (size_t)n * rb, K, wrow);
        for (int64_t m = 0; m < M; m++) {
            const float *xr = x + (size_t)m * K;
            double acc = 0.0;
            for (int64_t k = 0; k < K; k++) acc += (double)xr[k] * (double)wrow[k];
            if (bias) acc += (double)bias[n];   /* ml/ggml/dense.go:55-57 */
            y[(size_t)m * N + n] = gqo_activation(act, (float)acc); /* dense.go:58-60 */
        }
    }
    free(wrow);
    return 0;
}

int gqo_qdense_f32acc(int type, const float *x, int64_t M, int64_t K, const uint8_t *W,
                      int64_t N, const float *bias, int act, float *y, int threads) {
    block_fn fn = block_dequantizer(type);
    const size_t rb = gqo_row_bytes(type, K);
    if (!fn || rb == 0 || act < GQO_ACT_NONE || act > GQO_ACT_TANH) return -1;
    const int bpb = gqo_bytes_per_block(type), vpb = gqo_values_per_block(type);
    const int64_t nb = K / vpb;
    if (threads < 1) threads = 1;
#ifdef _OPENMP
#pragma omp parallel for num_threads(threads) schedule(static)
#endif
    for (int64_t n = 0; n < N; n++) {
        float blk[256];
        const uint8_t *row = W + (size_t)n * rb;
        for (int64_t m0 = 0; m0 < M; m0 += 8) { /* 8 activations share one pass over the row */
            const int mc = (int)((M - m0) < 8 ? (M - m0) : 8);
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int64_t b = 0; b < nb; b++) {
                fn(row + b * bpb, blk);
                for (int mi = 0; mi < mc; mi++) {
                    const float *xr = x + (size_t)(m0 + mi) * K + b * vpb;
                    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
                    for (int i = 0; i < vpb; i += 4) {
                        s0 += blk[i] * xr[i];
                        s1 += blk[i + 1] * xr[i + 1];
                        s2 += blk[i + 2] * xr[i + 2];
                        s3 += blk[i + 3] * xr[i + 3];
                    }
                    acc[mi] += (s0 + s1) + (s2 + s3);
                }
            }
            for (int mi = 0; mi < mc; mi++) {
                float v = acc[mi];
                if (bias) v += bias[n];
                y[(size_t)(m0 + mi) * N + n] = gqo_activation(act, v);
            }
        }
    }
    return 0;
}

/* ---- callers around the dense layers -------------------------------------- */

/* RMSNormBuilder.Done (ml/layers/norm/rmsnorm.go:78-113) over the last axis, node by node:
 * Square, ReduceMean (:86-87), AddScalar epsilon (:88-90), Sqrt (:91), Div (:92), and with a gain
 * AddScalar offset (:101-103), Mul (:111).  Each node's fp32 result is rounded on its own; the
 * mean is summed in double so that it is the correctly rounded mean whatever order a backend
 * reduces in. */
int gqo_rmsnorm(const float *x, int64_t M, int64_t K, const float *gain, float eps, float gain_offset,
                float *y) {
    if (M < 0 || K <= 0) return -1;
    for (int64_t m = 0; m < M; m++) {
        const float *xr = x + (size_t)m * K;
        float *yr = y + (size_t)m * K;
        double acc = 0.0;
        for (int64_t k = 0; k < K; k++) {
            const float sq = xr[k] * xr[k];
            acc += (double)sq;
        }
        float mean = (float)(acc / (double)K);
        if (eps != 0.0f) mean = mean + eps;
        const float rms = sqrtf(mean);
        for (int64_t k = 0; k < K; k++) {
            float v = xr[k] / rms;
            if (gain) {
                float g = gain[k];
                if (gain_offset != 0.0f) g = g + gain_offset;
                v = v * g;
            }
            yr[k] = v;
        }
    }
    return 0;
}

/* The gated feed-forward front of a decoder layer (ml/zoo/transformer/transformer.go:1276-1287):
 * x = normalize(x) when use_norm; gate = dense(x), up = dense(x); ff = Mul(activation(gate), up).
 * The projections are gqo_qdense (fp64 accumulation over the exact fp32 weights). */
int gqo_gated_ffn(int type, const float *x, int64_t M, int64_t K, int use_norm, const float *gain, float eps,
                  float gain_offset, const uint8_t *Wgate, const float *bias_gate, const uint8_t *Wup,
                  const float *bias_up, int64_t N, int act, float *y) {
    float *xn = NULL, *gate = (float *)malloc((size_t)(M * N > 0 ? M * N : 1) * sizeof(float));
    if (!gate) return -3;
    int rc = 0;
    if (use_norm) {
        xn = (float *)malloc((size_t)(M * K > 0 ? M * K : 1) * sizeof(float));
        if (!xn) { free(gate); return -3; }
        rc = gqo_rmsnorm(x, M, K, gain, eps, gain_offset, xn);
        x = xn;
    }
    if (!rc) rc = gqo_qdense(type, x, M, K, Wgate, N, bias_gate, act, gate);
    if (!rc) rc = gqo_qdense(type, x, M, K, Wup, N, bias_up, GQO_ACT_NONE, y);
    if (!rc)
        for (int64_t i = 0; i < M * N; i++) y[i] = gate[i] * y[i];
    free(gate);
    free(xn);
    return rc;
}

/* ---- gather ----------------------------------------------------------- */

int gqo_embedding_lookup(int type, const uint8_t *table, int64_t vocab, int64_t K,
                         const int32_t *indices, int64_t count, float *out) {
    block_fn fn = block_dequantizer(type);
    const size_t rb = gqo_row_bytes(type, K);
    if (!fn || rb == 0) return -1;
    const int bpb = gqo_bytes_per_block(type), vpb = gqo_values_per_block(type);
    for (int64_t i = 0; i < count; i++) {
        const int64_t r = indices[i];
        if (r < 0 || r >= vocab) return -2;
        dequant_row(fn, bpb, vpb, table + (size_t)r * rb, K, out + (size_t)i * K);
    }
    return 0;
}
