/*
 * Memory- and undefined-behaviour check of the CPU oracle (test infrastructure, like the oracle itself).
 *
 * Built together with ggml_oracle.c under -fsanitize=address,undefined (oracle/Makefile, target
 * oracle_selftest_asan) and run by tests/test_host_cpp.py.  Every function of ggml_oracle.h is called on
 * exactly-sized heap buffers (so a read or write one element past an end is caught), for every block format,
 * with all-random bytes in the weights (every bit pattern of the packed fields, non-finite scales included);
 * two of the reference's known answers (ml/nn/quantized_dense_test.go:277-305, 347-382) make sure the
 * instrumented build still computes the right thing.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "ggml_oracle.h"

static uint64_t state = 0x9E3779B97F4A7C15ull;
static uint32_t rnd(void) {
    state = state * 6364136223846793005ull + 1442695040888963407ull;
    return (uint32_t)(state >> 33);
}

static int failures = 0;
#define CHECK(cond, ...) do { if (!(cond)) { failures++; printf("FAIL %s:%d: ", __FILE__, __LINE__); printf(__VA_ARGS__); printf("\n"); } } while (0)

static void *exact(size_t bytes) {  /* (malloc(0) may return NULL: keep one byte) */
    void *p = malloc(bytes ? bytes : 1);
    if (!p) { printf("out of memory\n"); exit(2); }
    return p;
}

static void kats(void) {
    /* Q8_0: row0 = [2.0 | 1, 0 x31], row1 = [3.0 | 0, 1, 0 x30]; x = [1, 1, 0...] -> [2, 3] */
    uint8_t *W = exact(2 * 34);
    memset(W, 0, 2 * 34);
    W[1] = 0x40; W[2] = 1;
    W[34 + 1] = 0x42; W[34 + 3] = 1;
    float *x = exact(32 * sizeof(float)), *y = exact(2 * sizeof(float));
    memset(x, 0, 32 * sizeof(float));
    x[0] = x[1] = 1.f;
    CHECK(gqo_qdense(GQO_Q8_0, x, 1, 32, W, 2, NULL, GQO_ACT_NONE, y) == 0, "qdense status");
    CHECK(y[0] == 2.f && y[1] == 3.f, "Q8_0 known answer: %g %g", y[0], y[1]);
    free(W);
    /* Q4_0: byte 0x89 = low nibble 9 (+1 d at index j), high nibble 8 (0 at index j + 16) */
    W = exact(2 * 18);
    memset(W, 0x88, 2 * 18);
    W[0] = 0x00; W[1] = 0x40; W[2] = 0x89;
    W[18] = 0x00; W[19] = 0x42; W[21] = 0x89;
    CHECK(gqo_qdense(GQO_Q4_0, x, 1, 32, W, 2, NULL, GQO_ACT_NONE, y) == 0, "qdense status");
    CHECK(y[0] == 2.f && y[1] == 3.f, "Q4_0 known answer: %g %g", y[0], y[1]);
    free(W); free(x); free(y);
    CHECK(gqo_fp16_to_fp32(0x4000) == 2.f && gqo_fp16_to_fp32(0x4200) == 3.f && gqo_fp16_to_fp32(0x3C00) == 1.f, "fp16 known answers");
}

static void sweep(int type, int64_t K) {
    const int64_t N = 5, M = 3;
    const size_t rb = gqo_row_bytes(type, K);
    CHECK(rb > 0, "row bytes of type %d, K=%lld", type, (long long)K);
    uint8_t *W = exact(N * rb), *W2 = exact(N * rb);
    for (size_t i = 0; i < (size_t)N * rb; i++) { W[i] = (uint8_t)rnd(); W2[i] = (uint8_t)rnd(); }
    float *x = exact(M * K * sizeof(float)), *gain = exact(K * sizeof(float)), *bias = exact(N * sizeof(float));
    for (int64_t i = 0; i < M * K; i++) x[i] = (float)((int)(rnd() % 2001) - 1000) * 1e-3f;
    for (int64_t i = 0; i < K; i++) gain[i] = 1.f + (float)(rnd() % 100) * 1e-2f;
    for (int64_t i = 0; i < N; i++) bias[i] = (float)(rnd() % 7) - 3.f;
    float *deq = exact(N * K * sizeof(float)), *y = exact(M * N * sizeof(float)), *y2 = exact(M * N * sizeof(float));
    CHECK(gqo_dequantize(type, W, N, K, deq) == 0, "dequantize type %d", type);
    for (int act = GQO_ACT_NONE; act <= GQO_ACT_TANH; act++) {
        CHECK(gqo_qdense(type, x, M, K, W, N, act & 1 ? bias : NULL, act, y) == 0, "qdense type %d act %d", type, act);
        for (int threads = 1; threads <= 3; threads += 2)
            CHECK(gqo_qdense_f32acc(type, x, M, K, W, N, act & 1 ? bias : NULL, act, y2, threads) == 0, "f32acc type %d", type);
    }
    int32_t *idx = exact(4 * sizeof(int32_t));
    idx[0] = 0; idx[1] = (int32_t)N - 1; idx[2] = 2; idx[3] = 2;
    float *rows = exact(4 * K * sizeof(float));
    CHECK(gqo_embedding_lookup(type, W, N, K, idx, 4, rows) == 0, "lookup type %d", type);
    CHECK(memcmp(rows + K, deq + (N - 1) * K, K * sizeof(float)) == 0, "looked-up row differs from the dequantised one");
    idx[3] = (int32_t)N;
    CHECK(gqo_embedding_lookup(type, W, N, K, idx, 4, rows) == -2, "an index past the table must be reported");
    idx[3] = -1;
    CHECK(gqo_embedding_lookup(type, W, N, K, idx, 4, rows) == -2, "a negative index must be reported");
    float *xn = exact(M * K * sizeof(float));
    CHECK(gqo_rmsnorm(x, M, K, gain, 1e-5f, 0.f, xn) == 0, "rmsnorm");
    CHECK(gqo_rmsnorm(x, M, K, NULL, 1e-6f, 1.f, xn) == 0, "rmsnorm without gain");
    CHECK(gqo_gated_ffn(type, x, M, K, 1, gain, 1e-5f, 0.f, W, bias, W2, NULL, N, GQO_ACT_SILU, y) == 0, "gated ffn type %d", type);
    CHECK(gqo_gated_ffn(type, x, M, K, 0, NULL, 0.f, 0.f, W, NULL, W2, bias, N, GQO_ACT_GELU, y) == 0, "gated ffn type %d", type);
    /* empty problems touch nothing */
    CHECK(gqo_qdense(type, x, 0, K, W, N, NULL, 0, y) == 0 && gqo_qdense(type, x, M, K, W, 0, NULL, 0, y) == 0, "empty problems");
    CHECK(gqo_dequantize(type, W, N, K + 1, deq) == -1, "ragged K must be refused");
    free(W); free(W2); free(x); free(gain); free(bias); free(deq); free(y); free(y2); free(idx); free(rows); free(xn);
}

int main(void) {
    kats();
    const int types[] = {GQO_Q4_0, GQO_Q8_0, GQO_Q4_K, GQO_Q6_K, GQO_IQ4_NL};
    for (unsigned i = 0; i < sizeof(types) / sizeof(types[0]); i++) {
        const int vpb = gqo_values_per_block(types[i]);
        CHECK(vpb > 0 && gqo_bytes_per_block(types[i]) > 0, "block geometry of type %d", types[i]);
        for (int rep = 0; rep < 8; rep++) {
            sweep(types[i], vpb);
            sweep(types[i], 3 * (int64_t)vpb);
        }
    }
    CHECK(gqo_values_per_block(999) == 0 && gqo_bytes_per_block(999) == 0 && gqo_row_bytes(999, 256) == 0, "unknown type");
    for (int act = 0; act <= GQO_ACT_TANH; act++) {
        const float v = gqo_activation(act, -0.5f), big = gqo_activation(act, 1e30f), nbig = gqo_activation(act, -1e30f);
        CHECK(v == v && big == big && nbig == nbig, "activation %d gave NaN", act);
    }
    printf("%d failed\n", failures);
    return failures ? 1 : 0;
}
