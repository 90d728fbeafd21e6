/*
 * gomlx_hipq - MI355X (gfx950) implementation of GoMLX's quantized Dense hot path.
 *
 * C ABI of libgomlx_hipq.so.  A Go backend reaches it through cgo; every entry point
 * below names the interface of the reference (gomlx/gomlx, file:line) it stands in for.
 *
 * Conventions
 *   - Every function returns a gq_status (0 = success) unless stated otherwise; nothing
 *     throws or aborts across this boundary.  gq_last_error() returns the message of the
 *     last failure on the calling thread.
 *   - GQ_ERR_NOT_IMPLEMENTED is the analogue of compute.ErrNotImplemented: the caller may
 *     fall back to the decomposed graph (core/graph/fused_ops.go:357-363).  Any other
 *     error is a hard failure (core/graph/fused_ops.go:365).
 *   - All pointers named d* are device pointers owned by the caller; the library keeps no
 *     reference to them after the call returns (launches are asynchronous on `stream`, so
 *     the memory must stay valid until the stream has been synchronised).
 *   - Entry points are re-entrant.  Host threads that issue calls on the SAME stream are
 *     serialised for the length of one call's launches (multi-kernel paths share the stream's
 *     workspace); calls on different streams proceed independently.
 *   - stream == NULL selects the null stream of the active device.  Otherwise it is a
 *     hipStream_t.  The active device is the one given to gq_init(); every entry point
 *     makes it current on the calling thread itself (cgo may move a goroutine to another
 *     OS thread between calls).
 *   - Weights are native GGML blocks, row-major [N, gq_row_bytes(type, K)] bytes: one row
 *     per output feature, blocks running along K (ml/ggml/dense.go:19).
 *   - Activations x are row-major [M, K]; outputs y are row-major [M, N] fp32.
 */
#ifndef GOMLX_HIPQ_H
#define GOMLX_HIPQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    GQ_OK = 0,
    GQ_ERR_INVALID = 1,         /* malformed arguments: hard error */
    GQ_ERR_NOT_IMPLEMENTED = 2, /* valid but unsupported: caller may fall back */
    GQ_ERR_HIP = 3,             /* a HIP runtime call failed */
    GQ_ERR_NO_DEVICE = 4,       /* no usable gfx950 device / gq_init not called */
    GQ_ERR_OOM = 5
} gq_status;

/* compute.GGMLQuantType (core/graph/fused_ops.go:46-47); numeric values follow the public
 * GGML type ids. */
typedef enum { GQ_Q4_0 = 2, GQ_Q8_0 = 8, GQ_Q4_K = 12, GQ_Q6_K = 14, GQ_IQ4_NL = 20 } gq_type;

/* compute.ActivationType as produced by activation.Type.ToBackend
 * (ml/layers/activation/activation.go:58-75). */
typedef enum {
    GQ_ACT_NONE = 0, GQ_ACT_GELU = 1, GQ_ACT_RELU = 2, GQ_ACT_SILU = 3,
    GQ_ACT_HARDSWISH = 4, GQ_ACT_TANH = 5
} gq_act;

/* Activation element types accepted by the dense entry points. */
typedef enum { GQ_F32 = 0, GQ_BF16 = 1 } gq_dtype;

/* ABI version: bumped on any incompatible change. */
int gq_abi_version(void);

/* ---- geometry: GGMLQuantType.BytesPerBlock / ValuesPerBlock (ml/ggml/dequant.go:41,
 * ml/ggml/gather.go:24-25).  Pure host functions; return 0 for an unknown type. ---- */
int gq_bytes_per_block(int type);
int gq_values_per_block(int type);
/* (K / valuesPerBlock) * bytesPerBlock; 0 if the type is unknown or K is not a positive
 * whole number of blocks. */
size_t gq_row_bytes(int type, int64_t K);

/* ---- build-time validation: what Function.FusedQuantizedDense checks when the graph
 * is built (core/graph/fused_ops.go:195-245) and what Builder.OpShape then reports
 * (core/graph/fused_ops.go:238).  Needs no GPU.  On success *K_out receives the logical
 * feature count derived from w_row_bytes; the output shape is [M, N]. ---- */
int gq_qdense_check(int type, int x_dtype, int64_t M, int64_t x_last_dim, int64_t N,
                    int64_t w_row_bytes, int64_t bias_len /* -1: no bias */, int act,
                    int64_t *K_out);

/* ---- device, memory, streams: compute.Backend buffer plumbing
 * (BufferFromFlatData / ToFlatData, core/tensors/ondevice.go:273-285,462). ---- */
int gq_device_count(int *count);
int gq_init(int device);                 /* idempotent, thread-safe; requires gfx950 */
int gq_device_name(char *buf, size_t n);
int gq_malloc(void **dptr, size_t bytes);
int gq_free(void *dptr);
int gq_h2d(void *d, const void *h, size_t bytes, void *stream);  /* returns after the copy is done */
int gq_d2h(void *h, const void *d, size_t bytes, void *stream);  /* returns after the copy is done */
int gq_stream_create(void **stream);     /* default priority */
int gq_stream_destroy(void *stream);    /* waits for the stream and frees its workspaces */
int gq_sync(void *stream);

/* ---- ggml.Dequantize (ml/ggml/dequant.go:39-54): dW [N, row_bytes] -> dOut [N, K] fp32,
 * bit-exact with the reference arithmetic (one fp32 rounding per operation, no FMA). ---- */
int gq_dequantize(int type, const void *dW, int64_t N, int64_t K, float *dOut, void *stream);

/* ---- compute.Function.FusedQuantizedDense (core/graph/fused_ops.go:231-232), run time:
 * y = act(x . dequant(W)^T + bias), the contract of nn.QuantizedDense
 * (ml/nn/quantized_dense.go:31-57) and ggml.DenseDecomposed (ml/ggml/dense.go:23-62).
 * dBias may be NULL.  fp32 activations, fp32 accumulation.  The first few rows (4 to 6, depending
 * on format and matrix size; 16 for matrices of a few megabytes) run as bandwidth-bound GEMV
 * passes; larger batches contract on the matrix cores with the activations (and, from 65 to 385
 * rows on, depending on format and shape, the dequantised weights) rounded to fp16 operands (each batch row scaled by a power of two first, so the magnitude of x does not
 * matter).  Batches of 5 rows and more may use a
 * per-stream workspace that is created on the first such call on the stream: make
 * one call outside a recording (gq_graph_begin) before recording the same call. ---- */
int gq_qdense_f32(int type, const float *dX, int64_t M, int64_t K, const void *dW, int64_t N,
                  const float *dBias, int act, float *dY, void *stream);
/* gq_qdense_f32 for callers that cannot allocate device memory (code under HIP-graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same
 * arguments, same kernels and bit-identical results; the scratch memory that batches of 5 rows and
 * more use (activation image, split-K partial sums) is a fixed 16 MiB device array inside the library
 * instead of a per-stream workspace (its first 4 KiB are the flag words every workspace starts with:
 * 16 MiB - 4 KiB serve the call), and the call makes no hipMalloc / hipFree at all.  A problem
 * that needs more scratch than that (the two-pass GEMM's 16-bit weight image of a large matrix, or
 * about M * N * K / 2048 > 3.5 Mi for the split-K kernels) fails with GQ_ERR_INVALID and a message
 * naming the size; nothing is launched then.  Every call on a GPU shares that GPU's array: calls
 * that overlap in time on one GPU (different streams, or host threads that interleave) race; calls
 * on one stream from one thread are ordered and safe.  Not available while gq_profile_begin() is
 * active on the thread (event creation allocates). */
int gq_qdense_f32_static(int type, const float *dX, int64_t M, int64_t K, const void *dW, int64_t N,
                         const float *dBias, int act, float *dY, void *stream);
/* bf16 activations (raw 16-bit patterns), fp32 output.  Small batches widen the activations
 * exactly and take the same GEMV / split-K kernels as fp32 activations; beyond those batch
 * sizes the weights are dequantised to bf16 operands and contracted on bf16 MFMA with fp32 accumulation. */
int gq_qdense_bf16(int type, const uint16_t *dX, int64_t M, int64_t K, const void *dW,
                   int64_t N, const float *dBias, int act, float *dY, void *stream);

/* ---- Several FusedQuantizedDense nodes of one compiled graph that do not depend on each other
 * (e.g. the q/k/v or gate/up projections of a decoder layer) submitted together: the work an
 * Executable.Execute (core/graph/graph.go:669) is free to overlap.  Equivalent to calling
 * gq_qdense_f32 once per descriptor, in any order; outputs must not alias any input.  Batch-1
 * problems of one GGML type are merged into a single launch; two to four Q4_K projections of the
 * same activation buffer with 6 rows or more share one split-K pass (activations converted once). ---- */
typedef struct {
    int type;            /* gq_type */
    int act;             /* gq_act */
    const float *dX;     /* [M, K] */
    int64_t M, K;
    const void *dW;      /* [N, gq_row_bytes(type, K)] */
    int64_t N;
    const float *dBias;  /* [N] or NULL */
    float *dY;           /* [M, N] */
} gq_dense_desc;
int gq_qdense_f32_batch(int count, const gq_dense_desc *descs, void *stream);

/* ---- The callers on either side of the dense layers in a decoder block
 * (ml/zoo/transformer/transformer.go:1099-1101, 1275-1294).  These have no fused op in the
 * reference: a backend's Executable would recognise the node pattern. ----
 *
 * norm.RMSNorm(...).WithEpsilon(eps).WithScaleOffset(gain_offset).Done() over the last axis
 * (ml/layers/norm/rmsnorm.go:78-113): y = x / sqrt(mean(x^2) + eps) * (gain + gain_offset).
 * dGain [K] may be NULL (WithScale(false)). */
int gq_rmsnorm_f32(const float *dX, int64_t M, int64_t K, const float *dGain, float eps,
                   float gain_offset, float *dY, void *stream);
typedef struct {
    const float *dGain; /* [K] or NULL */
    float eps;
    float gain_offset;
} gq_rmsnorm;
/* A projection with its neighbours in the layer: y = residual + act(RMSNorm(x) . W^T + bias)
 * (Model.normalize followed by a projection, transformer.go:1099-1101; Add(residual, ...) after
 * the output and down projections, :1045, :1055, :1291-1292).  norm and dResidual may each be
 * NULL (both NULL is plain gq_qdense_f32); dY may be dResidual itself (a residual stream updated
 * in place).  Small batches (a few rows; up to 16 where the split-K kernels do not apply) run in
 * the decode GEMV itself when K is a multiple of 256 and x and gain are 16-byte aligned; large batches (those a plain call hands to the two-pass GEMM) fold the
 * normalisation into the activation pass and the residual into the GEMM epilogue; the batches in
 * between (split-K kernels) apply the gain where their activation image is written and the
 * division and the residual in their reduction; what is left is composed of an RMSNorm kernel,
 * the dense call and an addition.  All but the first use a per-stream workspace. */
int gq_qdense_block_f32(int type, const float *dX, int64_t M, int64_t K, const gq_rmsnorm *norm,
                        const void *dW, int64_t N, const float *dBias, int act,
                        const float *dResidual, float *dY, void *stream);
/* gq_qdense_f32_batch with one RMS normalisation applied to the activations of every problem:
 * the q/k/v projections behind a layer's input norm (transformer.go:1099-1130) in one launch
 * when all are problems of one type, one K and one batch size of at most 8 rows.  Two to four
 * Q4_K projections of the SAME activation buffer (equal dX, M, K) with more rows than that share
 * one split-K pass (activations converted once, one main launch, one reduction; uses the
 * per-stream workspace); past the split-K kernels' range such projections of any one type, with
 * widths that are multiples of 32 and one activation function, share the two-pass GEMM (one activation
 * conversion, one 16-bit image of all the matrices, one GEMM that writes each matrix's columns to its
 * own output); anything else runs as separate gq_qdense_block_f32 calls. */
int gq_qdense_norm_f32_batch(int count, const gq_dense_desc *descs, const gq_rmsnorm *norm,
                             void *stream);
/* The gated feed-forward front (transformer.go:1279-1287, after the pre_feedforward_norm of
 * :1276 when norm != NULL): y = act(xn . Wgate^T + bgate) * (xn . Wup^T + bup), xn = RMSNorm(x)
 * or x.  Both matrices are [N, gq_row_bytes(type, K)] of one type.  A few rows run as one launch
 * of the decode GEMV (conditions as for gq_qdense_block_f32); from 256 rows the two matrices are
 * dequantised into one interleaved 16-bit image and a single GEMM forms the product in
 * registers; in between, the split-K kernels contract both matrices against one activation
 * image in one launch (the normalisation in their pre-pass and reduction, the product in the
 * reduction) up to their batch limit, and dense calls are composed beyond it.  All but the
 * first use a per-stream workspace. */
int gq_qdense_gated_f32(int type, const float *dX, int64_t M, int64_t K, const gq_rmsnorm *norm,
                        const void *dWgate, const float *dBiasGate, const void *dWup,
                        const float *dBiasUp, int64_t N, int act, float *dY, void *stream);

/* The three calls above for bf16 activations (raw 16-bit patterns, 16-byte aligned; in the batched form every
 * descriptor's dX points at bf16 data): what the same layer code (transformer.go:1099-1101, 1276-1294) builds when the
 * model runs in bfloat16.  Gain, bias and residual stay fp32 and the result is fp32, as for gq_qdense_bf16.  Results
 * equal those of the fp32 entry points on the widened inputs bit for bit: the decode kernel and the split-K pre-pass read
 * the bf16 rows as they are and widen them in registers (exact), so a decode call costs what its fp32 twin costs; on the
 * other routes the activations are widened to fp32 in a per-stream workspace first - activation matrices shared by
 * several problems of a batch once - and then take the fp32 routes. */
int gq_qdense_block_bf16(int type, const uint16_t *dX, int64_t M, int64_t K, const gq_rmsnorm *norm,
                         const void *dW, int64_t N, const float *dBias, int act,
                         const float *dResidual, float *dY, void *stream);
int gq_qdense_norm_bf16_batch(int count, const gq_dense_desc *descs, const gq_rmsnorm *norm,
                              void *stream);
int gq_qdense_gated_bf16(int type, const uint16_t *dX, int64_t M, int64_t K, const gq_rmsnorm *norm,
                         const void *dWgate, const float *dBiasGate, const void *dWup,
                         const float *dBiasUp, int64_t N, int act, float *dY, void *stream);

/* ---- compute.Function.QuantizedEmbeddingLookup (core/graph/fused_ops.go:295-296;
 * nn.QuantizedGather ml/nn/quantized_gather.go:30-43; ml/ggml/gather.go:21-49):
 * dOut[i, :] = dequant(dTable[dIndices[i], :]), bit-exact.  An index outside [0, vocab)
 * yields a row of NaN and sets *dErrFlag (a device int32, may be NULL) to 1. ---- */
int gq_embedding_lookup(int type, const void *dTable, int64_t vocab, int64_t K,
                        const int32_t *dIndices, int64_t count, float *dOut,
                        int32_t *dErrFlag, void *stream);

/* ---- Executable.Execute of a compiled graph (core/graph/graph.go:669): a sequence of
 * launches recorded once and replayed with one submission (HIP graph).  Between begin
 * and end, entry points called with this stream are recorded, not run.  A graph replays on
 * the stream it was recorded on (its launches share that stream's workspace with eager calls,
 * in stream order); gq_graph_launch rejects any other.  The workspaces a graph points at
 * stay allocated until gq_graph_destroy, also after gq_stream_destroy. ---- */
int gq_graph_begin(void *stream);
int gq_graph_end(void *stream, void **graph_exec);
int gq_graph_launch(void *graph_exec, void *stream);
int gq_graph_destroy(void *graph_exec);

/* ---- kernel timing (the counterpart of the klog -v=1 wall clock around Execute,
 * core/graph/graph.go:667-671): while enabled on the calling thread, every kernel launch
 * is bracketed by HIP events on its own stream.  gq_profile_end waits for them and
 * reports the launch count and the summed kernel time. ---- */
int gq_profile_begin(void);
int gq_profile_end(int *launches, double *total_us);

/* Bookkeeping of the per-stream workspaces (no counterpart in the reference; for tests and for callers that
 * watch device memory): the bytes the library currently holds for them and the number of streams that own one.
 * Either pointer may be null.  The fixed array of gq_qdense_f32_static is not counted. */
int gq_workspace_stats(size_t *live_bytes, int *streams);

/* Message of the last error on this thread; valid until the next failing call. */
const char *gq_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
