// The callers on either side of a quantized dense layer in a decoder block
// (ml/zoo/transformer/transformer.go:1275-1294): the RMS normalisation in front of the
// projections (ml/layers/norm/rmsnorm.go:78-113) and the gated feed-forward front
//     ff = act(x . Wgate^T + bgate) * (x . Wup^T + bup).
//
// For a few activation rows both are folded into the K-sliced decode GEMV (gemv_ks_body.hpp,
// EXT): one launch reads the two weight matrices once and writes only ff.  Larger batches are
// composed from the dense kernels plus the small kernels below.
#include "gemv_ks_body.hpp"

namespace gq {

namespace {

// X: fp32, or bf16 with XBF16 (widened while a slice is converted: exact)
template <int T, int PF, int WIN, int R, bool XBF16>
__global__ __launch_bounds__(512) void gemv_ks_ext_kernel(const void *__restrict__ X, const uint8_t *__restrict__ W,
                                                          const float *__restrict__ bias, float *__restrict__ Y, int M, int K, int N,
                                                          int64_t row_bytes, int iters, int nslices, int half_tail, int act,
                                                          const KsExt ext) {
    extern __shared__ uint32_t lds[];
    const int r0 = (int)blockIdx.y * R;
    KsExt e = ext;
    if (e.residual) e.residual += (int64_t)r0 * N;
    const int64_t x_stride = (int64_t)K * (XBF16 ? 2 : 4);
    ks_body<T, PF, WIN, true, XBF16, R>(reinterpret_cast<const uint8_t *>(X) + r0 * x_stride, W, bias, Y + (int64_t)r0 * N, N, row_bytes, iters, nslices,
                                        half_tail, act, (int)(blockDim.x >> 6), (int)blockIdx.x, lds, &e, min(R, M - r0), x_stride, 0, (int)gridDim.x);
}

// Batched submission (several batch-1 projections of one format in one launch) with one RMS
// normalisation shared by all of them: the q/k/v projections behind a layer's input norm.
template <int T, bool XBF16>
__global__ __launch_bounds__(512) void gemv_ks_batch_ext_kernel(const KsBatch b, const KsExt ext) {
    extern __shared__ uint32_t lds[];
    const KsProblem &q = b.p[ks_batch_problem(b, (int)blockIdx.x)];
    const int64_t row = blockIdx.y;  // activation row of every problem
    const uint8_t *x = reinterpret_cast<const uint8_t *>(q.x) + row * q.K * (XBF16 ? 2 : 4);  // (q.x points at bf16 data with XBF16)
    ks_body<T, kBatchPF, kBatchWin, true, XBF16, 1, true>(x, q.W, q.bias, q.y + row * q.N, q.N, q.row_bytes, q.iters, q.nslices, q.half_tail, q.act, q.waves,
                                                (int)blockIdx.x - q.wg_begin, lds, &ext, 1, 0, q.live, q.nwg);
}

template <int T>
int launch_batch_ext(int count, const XsBatchItem *items, const KsExt &ext, int rows, bool x_is_bf16, hipStream_t s) {
    KsBatch b;
    size_t shmem;
    int wgs;
    if (int rc = plan_ks_batch<T>(count, items, b, shmem, wgs)) return rc;
    if (x_is_bf16) return launch(gemv_ks_batch_ext_kernel<T, true>, dim3((unsigned)wgs, (unsigned)rows), dim3(512), shmem, s, b, ext);
    return launch(gemv_ks_batch_ext_kernel<T, false>, dim3((unsigned)wgs, (unsigned)rows), dim3(512), shmem, s, b, ext);
}

template <int T, int PF, int R = 1>
int launch_ext_pf(const KsPlan &p, const void *x, bool x_is_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
                  const KsExt &ext, hipStream_t s) {
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    const dim3 grid((unsigned)p.wgs, (unsigned)((M + R - 1) / R)), block((unsigned)p.waves * 64);
    constexpr int WIN = PF < 3 ? PF : 3;
    if (x_is_bf16)
        return launch(gemv_ks_ext_kernel<T, PF, WIN, R, true>, grid, block, ks_lds_bytes(p.waves, p.iters, R), s, x, W, bias, y, (int)M, (int)K, (int)N,
                      row_bytes, p.iters, p.nslices, p.half_tail, act, ext);
    return launch(gemv_ks_ext_kernel<T, PF, WIN, R, false>, grid, block, ks_lds_bytes(p.waves, p.iters, R), s, x, W, bias, y, (int)M, (int)K, (int)N,
                  row_bytes, p.iters, p.nslices, p.half_tail, act, ext);
}

template <int T, int R>
int launch_ext_rows(KsPlan p, bool dual, const void *x, bool x_is_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
                    const KsExt &ext, hipStream_t s) {
    ks_regroup(p, N, dual, 4);  // (two alternating matrices: 2 or 4, both even)
    switch (p.pf) {
    case 1: return launch_ext_pf<T, 1, R>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case 2: return launch_ext_pf<T, 2, R>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    default: return launch_ext_pf<T, 4, R>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    }
}

template <int T>
int launch_ext(const void *x, bool x_is_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y, const KsExt &ext,
               hipStream_t s) {
    // With two matrices the row-steps alternate between them: plan for 2 N rows and an even count.
    const bool dual = ext.W2 != nullptr;
    KsPlan p;
    if (!ks_plan(K, dual ? 2 * N : N, p, dual)) return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv_ks: unsupported problem");
    if (dual) p.wgs = (int)((N + p.iters * 4 - 1) / (p.iters * 4));
    // batches over a large matrix run as passes of two rows (the extras leave no registers for the planes of four)
    if (M >= 2 && (int64_t)gq_row_bytes(T, K) * N * (dual ? 2 : 1) >= kLargeWeightBytes)
        return launch_ext_rows<T, 2>(p, dual, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    switch (p.pf) {
    case 1: return launch_ext_pf<T, 1>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case 2: return launch_ext_pf<T, 2>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case 3: return launch_ext_pf<T, 3>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case 4: return launch_ext_pf<T, 4>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case 5: return launch_ext_pf<T, 5>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case 6: return launch_ext_pf<T, 6>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case 7: return launch_ext_pf<T, 7>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    default: return launch_ext_pf<T, 8>(p, x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    }
}

// y = x / sqrt(mean(x^2) + eps) * (gain + offset), one workgroup per row (the operations and their
// order follow ml/layers/norm/rmsnorm.go:86-111: Square, ReduceMean, AddScalar, Sqrt, Div, Mul).
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float *__restrict__ X, const float *__restrict__ gain, float gain_offset, float eps,
                                                      int K, float *__restrict__ Y) {
    __shared__ float part[4];
    const float *x = X + (int64_t)blockIdx.x * K;
    float *y = Y + (int64_t)blockIdx.x * K;
    float ss = 0.f;
    for (int k = threadIdx.x; k < K; k += 256) ss = fmaf(x[k], x[k], ss);
    for (int m = 1; m < 64; m <<= 1) ss += __shfl_xor(ss, m);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float mean = ((part[0] + part[1]) + (part[2] + part[3])) / (float)K;
    const float r = sqrtf(mean + eps);
    for (int k = threadIdx.x; k < K; k += 256) {
        float v = x[k] / r;
        if (gain) v *= gain[k] + gain_offset;
        y[k] = v;
    }
}

// y[i] = a[i] + r[i]; y may be a or r (one thread per element)
__global__ __launch_bounds__(256) void add_kernel(const float *a, const float *r, float *y, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = a[i] + r[i];
}

// y[i] = x[i] widened from bf16 (exact: a shift); eight values per thread, n % 8 == 0 handled by the caller's padding rule
__global__ __launch_bounds__(256) void widen_bf16_kernel(const uint16_t *__restrict__ x, float *__restrict__ y, int64_t n) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i + 8 <= n) {
        const uint4 v = *reinterpret_cast<const uint4 *>(x + i);
        float4 lo = make_float4(bf16_lo(v.x), bf16_hi(v.x), bf16_lo(v.y), bf16_hi(v.y));
        float4 hi = make_float4(bf16_lo(v.z), bf16_hi(v.z), bf16_lo(v.w), bf16_hi(v.w));
        *reinterpret_cast<float4 *>(y + i) = lo;
        *reinterpret_cast<float4 *>(y + i + 4) = hi;
    } else {
        for (int64_t j = i; j < n; j++) y[j] = __builtin_bit_cast(float, (uint32_t)x[j] << 16);
    }
}

// y[i] *= g[i]
__global__ __launch_bounds__(256) void mul_inplace_kernel(float *__restrict__ y, const float *__restrict__ g, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] *= g[i];
}

}  // namespace

bool gemv_ks_ext_supported(int type, int64_t M, int64_t K, int64_t N, const void *x, const void *gain) {
    if (M < 1 || M > 16 || N > (int64_t)INT32_MAX / 8) return false;
    if (gain && (reinterpret_cast<uintptr_t>(gain) & 15)) return false;
    return gemv_ks_supported(type, K, N, x);
}

namespace {
KsExt make_ext(const RmsNorm *norm, int64_t K, const uint8_t *W2, const float *bias2, const float *residual) {
    KsExt ext = {};
    ext.W2 = W2;
    ext.bias2 = bias2;
    ext.residual = residual;
    if (norm) {
        ext.norm = 1;
        ext.gain = norm->gain;
        ext.gain_offset = norm->gain_offset;
        ext.eps = norm->eps;
        ext.inv_k = 1.0f / (float)K;
    }
    return ext;
}
}  // namespace

int launch_gemv_ks_ext(int type, const void *x, bool x_is_bf16, int64_t M, int64_t K, const RmsNorm *norm, const uint8_t *W, const float *bias,
                       const uint8_t *W2, const float *bias2, const float *residual, int64_t N, int act, float *y, hipStream_t s) {
    const KsExt ext = make_ext(norm, K, W2, bias2, residual);
    switch (type) {
    case kQ4_0: return launch_ext<kQ4_0>(x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case kQ8_0: return launch_ext<kQ8_0>(x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case kQ4_K: return launch_ext<kQ4_K>(x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case kQ6_K: return launch_ext<kQ6_K>(x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    case kIQ4_NL: return launch_ext<kIQ4_NL>(x, x_is_bf16, M, K, W, N, bias, act, y, ext, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv_ks: ggml type %d is not implemented", type);
    }
}

// all problems share K (one normalised input feeds them)
int launch_gemv_ks_batch_norm(int type, int count, const XsBatchItem *items, const RmsNorm *norm, hipStream_t s, int rows, bool x_is_bf16) {
    if (count < 1 || count > kMaxBatchKs) return fail(GQ_ERR_INVALID, "gemv batch: %d problems (1..%d supported per launch)", count, kMaxBatchKs);
    const KsExt ext = make_ext(norm, items[0].K, nullptr, nullptr, nullptr);
    switch (type) {
    case kQ4_0: return launch_batch_ext<kQ4_0>(count, items, ext, rows, x_is_bf16, s);
    case kQ8_0: return launch_batch_ext<kQ8_0>(count, items, ext, rows, x_is_bf16, s);
    case kQ4_K: return launch_batch_ext<kQ4_K>(count, items, ext, rows, x_is_bf16, s);
    case kQ6_K: return launch_batch_ext<kQ6_K>(count, items, ext, rows, x_is_bf16, s);
    case kIQ4_NL: return launch_batch_ext<kIQ4_NL>(count, items, ext, rows, x_is_bf16, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv batch: ggml type %d is not implemented", type);
    }
}

int launch_add(const float *a, const float *r, float *y, int64_t n, hipStream_t s) {
    return launch(add_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, a, r, y, n);
}

int launch_rmsnorm(const float *x, int64_t M, int64_t K, const float *gain, float gain_offset, float eps, float *y, hipStream_t s) {
    return launch(rmsnorm_kernel, dim3((unsigned)M), dim3(256), 0, s, x, gain, gain_offset, eps, (int)K, y);
}

int launch_widen_bf16(const uint16_t *x, float *y, int64_t n, hipStream_t s) {
    if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(y) & 15)) return fail(GQ_ERR_INVALID, "bf16 activations must be 16-byte aligned");
    return launch(widen_bf16_kernel, dim3((unsigned)((n + 2047) / 2048)), dim3(256), 0, s, x, y, n);
}

int launch_mul_inplace(float *y, const float *g, int64_t n, hipStream_t s) {
    return launch(mul_inplace_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, y, g, n);
}

}  // namespace gq
