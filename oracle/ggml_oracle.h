/*
 * CPU oracle for GoMLX's quantized Dense path (GGML block formats).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke
 * check and the benchmark's CPU-baseline leg may link or call it; the GPU library
 * never does.  Every function restates, in plain scalar C, the algorithm of the
 * reference (gomlx/gomlx) at the cited file:line.
 *
 * Pinning status (what fixes each function's results independently of this file):
 *   gqo_fp16_to_fp32      pinned  - exhaustive comparison with IEEE binary16 (numpy) + reference KATs
 *   Q8_0 / Q4_0 dequant   pinned  - ml/nn/quantized_dense_test.go:272-401 KATs, closed form, brute force
 *   IQ4_NL dequant        pinned  - ml/nn/quantized_dense_test.go:406-452 KAT (LUT[8]=1, LUT[9]=13) + public table
 *   dense / bias / act    pinned  - reference KATs, unit-vector probes, linearity, SiLU KAT, the activation vectors
 *                                   of ml/layers/activation/activation_test.go:17-112
 *   gather                pinned  - ml/nn/quantized_gather_test.go:17-169 KATs
 *   RMS normalisation     pinned  - ml/layers/norm/rmsnorm_test.go:16-45 KAT, closed forms (constant rows,
 *                                   scale invariance, unit norm), independent numpy form
 *   gated feed-forward    pinned  - composition of the pinned parts (two dense products, activation, Mul),
 *                                   checked against that composition written out in numpy
 *   Q4_K dequant          PARITY UNPINNED at the reference: the only implementation lives in the
 *                         third-party module github.com/gomlx/compute v0.1.2 (package gobackend),
 *                         which is not vendored.  Restated from the public GGML block_q4_K
 *                         specification.  What stays open is the BYTE LAYOUT only: given the fields,
 *                         the value is fixed by the mathematics - d*sc, (d*sc)*q, d*(sc*q) and dmin*m
 *                         are exact in binary32, so w = fl(d*sc*q - dmin*m) is one correctly rounded
 *                         subtraction under every order of operations, with or without a fused
 *                         multiply-add (checked against exact rationals rounded once).
 *   Q6_K dequant          PARITY UNPINNED at the reference, for the same reason (the reference names
 *                         the type, docs/CHANGELOG.md:251-252, but holds neither its arithmetic nor a
 *                         test vector).  Restated from the public GGML block_q6_K specification;
 *                         exact-arithmetic and structural checks only.
 */
#ifndef GGML_ORACLE_H
#define GGML_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGML type ids (public ggml numbering). */
enum { GQO_Q4_0 = 2, GQO_Q8_0 = 8, GQO_Q4_K = 12, GQO_Q6_K = 14, GQO_IQ4_NL = 20 };

/* compute.ActivationType as used by activation.Type.ToBackend
 * (ml/layers/activation/activation.go:58-75). */
enum { GQO_ACT_NONE = 0, GQO_ACT_GELU = 1, GQO_ACT_RELU = 2, GQO_ACT_SILU = 3,
       GQO_ACT_HARDSWISH = 4, GQO_ACT_TANH = 5 };

/* IEEE-754 binary16 -> binary32, exact (Bitcast u8[2]->f16 little-endian then
 * ConvertDType, ml/ggml/dequant.go:63-66). */
float gqo_fp16_to_fp32(uint16_t h);

/* GGMLQuantType.BytesPerBlock / ValuesPerBlock (used at ml/ggml/dequant.go:41,
 * ml/ggml/gather.go:24-25).  Return 0 for unknown types. */
int gqo_bytes_per_block(int type);
int gqo_values_per_block(int type);
/* (K / valuesPerBlock) * bytesPerBlock, or 0 if K is not a whole number of blocks. */
size_t gqo_row_bytes(int type, int64_t K);

/* ggml.Dequantize (ml/ggml/dequant.go:39-54): W [N, rowBytes] u8 -> out [N, K] f32.
 * Returns 0 on success, -1 for an unsupported type or ragged K. */
int gqo_dequantize(int type, const uint8_t *W, int64_t N, int64_t K, float *out);

/* nn.QuantizedDense GGML branch (ml/nn/quantized_dense.go:47-57) =
 * ggml.DenseDecomposed (ml/ggml/dense.go:23-62): y = act(x . dequant(W)^T + bias).
 * x [M,K] f32, W [N,rowBytes] u8, bias [N] or NULL, y [M,N] f32.
 * Products of the exact fp32 weights with x are accumulated in fp64 and rounded
 * once: this is the gold value the GPU outputs are compared against. */
int gqo_qdense(int type, const float *x, int64_t M, int64_t K, const uint8_t *W,
               int64_t N, const float *bias, int act, float *y);

/* Same contract as gqo_qdense, but computed the way a CPU backend would run it:
 * block-streamed dequantization fused with an fp32 dot product, `threads` OpenMP
 * threads over output rows.  Used only as the timed CPU baseline. */
int gqo_qdense_f32acc(int type, const float *x, int64_t M, int64_t K, const uint8_t *W,
                      int64_t N, const float *bias, int act, float *y, int threads);

/* ggml.EmbeddingLookupDecomposed (ml/ggml/gather.go:21-49): out[i,:] =
 * dequant(table[indices[i], :]).  Returns -2 if an index is out of range. */
int gqo_embedding_lookup(int type, const uint8_t *table, int64_t vocab, int64_t K,
                         const int32_t *indices, int64_t count, float *out);

/* norm.RMSNorm over the last axis (ml/layers/norm/rmsnorm.go:78-113):
 * y = x / sqrt(mean(x^2) + eps) * (gain + gain_offset); gain [K] or NULL (WithScale(false)). */
int gqo_rmsnorm(const float *x, int64_t M, int64_t K, const float *gain, float eps, float gain_offset,
                float *y);

/* Gated feed-forward front (ml/zoo/transformer/transformer.go:1276-1287):
 * y = act(xn . Wgate^T + bias_gate) * (xn . Wup^T + bias_up), xn = RMSNorm(x) if use_norm else x. */
int gqo_gated_ffn(int type, const float *x, int64_t M, int64_t K, int use_norm, const float *gain, float eps,
                  float gain_offset, const uint8_t *Wgate, const float *bias_gate, const uint8_t *Wup,
                  const float *bias_up, int64_t N, int act, float *y);

/* Epilogue of the fused op on one value (activation.Apply formulas,
 * ml/layers/activation/activation.go:161,195,222-243,274-286). */
float gqo_activation(int act, float v);

#ifdef __cplusplus
}
#endif
#endif
