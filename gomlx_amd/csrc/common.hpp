// Host-side plumbing shared by the translation units of libgomlx_hipq.so: status codes,
// thread-local error text, the active device, and the single kernel-launch path (which is
// where per-kernel event timing hooks in).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "../../include/gomlx_hipq.h"

namespace gq {

// ---- error text -----------------------------------------------------------------------
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t e, const char *what);

#define GQ_HIP(call)                                          \
    do {                                                      \
        hipError_t e__ = (call);                              \
        if (e__ != hipSuccess) return ::gq::hip_fail(e__, #call); \
    } while (0)

// ---- device ---------------------------------------------------------------------------
// Makes the device chosen by gq_init() current on this thread; fails if gq_init() has not
// succeeded yet.
int use_device();
int device_cu_count();

// ---- per-stream scratch memory (grows on demand; must exist before a graph recording uses it) ----
// Slot 0 belongs to the dense kernels, slot 1 to the operations composed of several dense calls.
// Every buffer is preceded by kWsSyncBytes of flag words (`sync`, if asked for) that are zero when the buffer is
// created; kernels that use them leave them zero again.
constexpr size_t kWsSyncBytes = 4096;
int stream_workspace(hipStream_t s, size_t bytes, void **out, int slot = 0, uint32_t **sync = nullptr);

// ---- launch ---------------------------------------------------------------------------
struct ProfileState {
    bool active = false;
    std::vector<hipEvent_t> events;  // start/stop pairs of the launches made while active
};
ProfileState &profile_state();

// Launches `kernel`; while profiling is active on this thread the launch carries a
// start/stop event pair whose timestamps are the kernel's own begin and end.
template <typename... KArgs, typename... Args>
int launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t shmem, hipStream_t stream, Args... args) {
    ProfileState &ps = profile_state();
    if (ps.active) {
        hipEvent_t a, b;
        GQ_HIP(hipEventCreate(&a));
        GQ_HIP(hipEventCreate(&b));
        hipExtLaunchKernelGGL(kernel, grid, block, (unsigned)shmem, stream, a, b, 0, static_cast<KArgs>(args)...);
        ps.events.push_back(a);
        ps.events.push_back(b);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, (unsigned)shmem, stream, static_cast<KArgs>(args)...);
    }
    GQ_HIP(hipGetLastError());
    return GQ_OK;
}

// Weight matrices from this size on count as large where kernels choose by size (batched GEMV passes, split-K crossovers).
constexpr int64_t kLargeWeightBytes = (int64_t)24 << 20;

// ---- kernel families (one translation unit each) -----------------------------------------
int launch_dequantize(int type, const uint8_t *W, int64_t N, int64_t K, float *out, hipStream_t s);
int launch_embedding_lookup(int type, const uint8_t *table, int64_t vocab, int64_t K, const int32_t *idx,
                            int64_t count, float *out, int32_t *err_flag, hipStream_t s);
int launch_gemv(int type, const float *x, int64_t M, int64_t K, const uint8_t *W, int64_t N,
                const float *bias, int act, float *y, hipStream_t s);
bool gemv_xs_supported(int type, int64_t K, int64_t N, const void *x);
int launch_gemv_xs(int type, const float *x, int64_t M, int64_t K, const uint8_t *W, int64_t N,
                   const float *bias, int act, float *y, hipStream_t s);
bool gemv_ks_supported(int type, int64_t K, int64_t N, const void *x);
int launch_gemv_ks(int type, const void *x, bool x_is_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N,
                   const float *bias, int act, float *y, hipStream_t s);
bool mmq_supported(int type, int64_t M, int64_t K, int64_t N, const void *x, const void *bias, const void *y);
// RMS normalisation in front of a projection: x / sqrt(mean(x^2) + eps) * (gain + gain_offset); gain may be null.
struct RmsNorm { const float *gain; float eps, gain_offset; };
// Optional extras of a split-K call: a second matrix (the result becomes act(x.W + bias) * (x.W2 + bias2), both
// contracted against one activation image and combined in the reduction), a residual added last, and an RMS
// normalisation of the (fp32) activations (gain 16-byte aligned or null): the gain is applied where the activation
// image is written, the division by the root mean square in the reduction.
struct MmqExtra { const uint8_t *W2; const float *bias2; const float *residual; const RmsNorm *norm; };
int launch_mmq(int type, const void *x, bool x_is_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias,
               int act, float *y, hipStream_t s, const MmqExtra *ex = nullptr);
// Several matrices of one K contracted against the same activations (fp32 or bf16 [M, K]) in one split-K pass: one
// activation pre-pass, one main launch over all their rows, one reduction (Q4_K; 2 to 4 matrices, each as mmq_supported asks).
struct MmqSetItem { const uint8_t *W; int64_t N; const float *bias; int act; float *y; };
bool mmq_set_supported(int type, int count, const MmqSetItem *items, int64_t M, int64_t K, const void *x);
int launch_mmq_set(int type, const void *x, bool x_is_bf16, int64_t M, int64_t K, int count, const MmqSetItem *items, const RmsNorm *norm,
                   hipStream_t s);
// The K-sliced GEMV with the normalisation folded in and, when W2 is given, the gated product
// act(x.W + bias) * (x.W2 + bias2); fp32 or bf16 activations, at most 16 rows (the entry points use it below 8 rows, where a pass per row still wins).
bool gemv_ks_ext_supported(int type, int64_t M, int64_t K, int64_t N, const void *x, const void *gain);
int launch_gemv_ks_ext(int type, const void *x, bool x_is_bf16, int64_t M, int64_t K, const RmsNorm *norm, const uint8_t *W, const float *bias,
                       const uint8_t *W2, const float *bias2, const float *residual, int64_t N, int act, float *y, hipStream_t s);
int launch_add(const float *a, const float *r, float *y, int64_t n, hipStream_t s);
int launch_rmsnorm(const float *x, int64_t M, int64_t K, const float *gain, float gain_offset, float eps, float *y, hipStream_t s);
int launch_mul_inplace(float *y, const float *g, int64_t n, hipStream_t s);
int launch_widen_bf16(const uint16_t *x, float *y, int64_t n, hipStream_t s);  // bf16 -> fp32 (exact); both 16-byte aligned
struct XsBatchItem { const float *x; const uint8_t *W; const float *bias; float *y; int64_t K, N; int act; };
int launch_gemv_xs_batch(int type, int count, const XsBatchItem *items, hipStream_t s);
// (K-sliced: `rows` activation rows per problem, the same count for all: x and y are [rows, K] and [rows, N])
int launch_gemv_ks_batch(int type, int count, const XsBatchItem *items, hipStream_t s, int rows = 1);
// the same with one RMS normalisation applied to every problem's activations (all of one K)
int launch_gemv_ks_batch_norm(int type, int count, const XsBatchItem *items, const RmsNorm *norm, hipStream_t s, int rows = 1, bool x_is_bf16 = false);
// Large batches: dequantise W once into a 16-bit image (in `workspace`, gemm_two_pass_workspace()
// bytes), then a plain 16-bit MFMA GEMM.
bool gemm_two_pass_supported(int type, bool x_is_bf16, int64_t M, int64_t K, int64_t N, const void *x);
size_t gemm_two_pass_workspace(bool x_is_bf16, int64_t M, int64_t K, int64_t N);
int launch_gemm_two_pass(int type, bool x_is_bf16, const void *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias,
                         int act, float *y, void *workspace, hipStream_t s);
// The two passes with the neighbours of a projection folded in (fp32 activations; same conditions as
// gemm_two_pass_supported): RMS normalisation in the activation pass, residual in the GEMM epilogue;
// with W2 one GEMM over the interleaved image of both matrices forms the gated product in registers.
size_t gemm_two_pass_block_workspace(int64_t M, int64_t K, int64_t N, bool gated);
bool gemm_two_pass_block_supported(int type, int64_t M, int64_t K, int64_t N, const void *x, bool gated);
int launch_gemm_two_pass_block(int type, const float *x, int64_t M, int64_t K, const RmsNorm *norm, const uint8_t *W, const float *bias,
                               const uint8_t *W2, const float *bias2, const float *residual, int64_t N, int act, float *y, void *workspace,
                               hipStream_t s);
// Two to four matrices against the same fp32 activations through the two passes: one activation conversion, one image, one
// GEMM that writes each matrix's columns to its own output (every N a multiple of 32, one activation for all).
bool gemm_two_pass_set_supported(int type, int count, const MmqSetItem *items, int64_t M, int64_t K, const void *x);
size_t gemm_two_pass_set_workspace(int count, const MmqSetItem *items, int64_t M, int64_t K);
int launch_gemm_two_pass_set(int type, const float *x, int64_t M, int64_t K, const RmsNorm *norm, int count, const MmqSetItem *items, void *workspace,
                             hipStream_t s);
int launch_gemm(int type, bool x_is_bf16, const void *x, int64_t M, int64_t K, const uint8_t *W, int64_t N,
                const float *bias, int act, float *y, hipStream_t s);

}  // namespace gq
