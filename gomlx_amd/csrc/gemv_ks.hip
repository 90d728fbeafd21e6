// Decode GEMV, K-sliced integer-dot kernels (Q4_0, Q8_0, Q4_K, Q6_K, IQ4_NL; K % 256 == 0): the
// kernels and launchers of the plain dense call and of batched submission.  The work of a
// workgroup is in gemv_ks_body.hpp.
#include "gemv_ks_body.hpp"

namespace gq {

namespace {

template <int T, int PF, int WIN, bool XBF16>
__global__ __launch_bounds__(512) void gemv_ks_kernel(const void *__restrict__ X, const uint8_t *__restrict__ W,
                                                      const float *__restrict__ bias, float *__restrict__ Y, int K, int N,
                                                      int64_t row_bytes, int iters, int nslices, int half_tail, int act) {
    extern __shared__ uint32_t lds[];
    const uint8_t *x = reinterpret_cast<const uint8_t *>(X) + (int64_t)blockIdx.y * K * (XBF16 ? 2 : 4);
    ks_body<T, PF, WIN, false, XBF16>(x, W, bias, Y + (int64_t)blockIdx.y * N, N, row_bytes, iters, nslices, half_tail, act, (int)(blockDim.x >> 6),
                        (int)blockIdx.x, lds);
}

template <int T>
__global__ __launch_bounds__(512) void gemv_ks_batch_kernel(const KsBatch b) {
    extern __shared__ uint32_t lds[];
    const KsProblem &q = b.p[ks_batch_problem(b, (int)blockIdx.x)];
    ks_body<T, kBatchPF, kBatchPF>(q.x, q.W, q.bias, q.y, q.N, q.row_bytes, q.iters, q.nslices, q.half_tail, q.act, q.waves,
                     (int)blockIdx.x - q.wg_begin, lds);
}


template <int T, int PF>
int launch_ks_pf(const KsPlan &p, const void *x, int x_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act,
                 float *y, hipStream_t s) {
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    const dim3 grid((unsigned)p.wgs, (unsigned)M), block((unsigned)p.waves * 64);
    constexpr int WIN = PF < 3 ? PF : 3;
    if (x_bf16)
        return launch(gemv_ks_kernel<T, PF, WIN, true>, grid, block, p.shmem, s, x, W, bias, y, (int)K, (int)N, row_bytes, p.iters, p.nslices,
                      p.half_tail, act);
    return launch(gemv_ks_kernel<T, PF, WIN, false>, grid, block, p.shmem, s, x, W, bias, y, (int)K, (int)N, row_bytes, p.iters, p.nslices,
                  p.half_tail, act);
}

template <int T>
int launch_ks(const void *x, int x_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
              hipStream_t s) {
    KsPlan p;
    if (!ks_plan(K, N, p)) return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv_ks: unsupported problem");
    switch (p.pf) {
    case 1: return launch_ks_pf<T, 1>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    case 2: return launch_ks_pf<T, 2>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    case 3: return launch_ks_pf<T, 3>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    case 4: return launch_ks_pf<T, 4>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    case 5: return launch_ks_pf<T, 5>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    case 6: return launch_ks_pf<T, 6>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    case 7: return launch_ks_pf<T, 7>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    default: return launch_ks_pf<T, 8>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    }
}

template <int T>
int launch_ks_batch(int count, const XsBatchItem *items, hipStream_t s) {
    KsBatch b;
    size_t shmem;
    int wgs;
    if (int rc = plan_ks_batch<T>(count, items, b, shmem, wgs)) return rc;
    return launch(gemv_ks_batch_kernel<T>, dim3((unsigned)wgs), dim3(512), shmem, s, b);
}

}  // namespace

bool gemv_ks_supported(int type, int64_t K, int64_t N, const void *x) {
    if (reinterpret_cast<uintptr_t>(x) & 15) return false;
    if (type != kQ4_0 && type != kQ8_0 && type != kQ4_K && type != kQ6_K && type != kIQ4_NL) return false;
    if (N <= 0 || N > (int64_t)INT32_MAX / 2) return false;
    int waves, nslices, half_tail;
    return ks_split(K, waves, nslices, half_tail);
}

int launch_gemv_ks(int type, const void *x, bool x_is_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias,
                   int act, float *y, hipStream_t s) {
    const int x_bf16 = x_is_bf16 ? 1 : 0;
    switch (type) {
    case kQ4_0: return launch_ks<kQ4_0>(x, x_bf16, M, K, W, N, bias, act, y, s);
    case kQ8_0: return launch_ks<kQ8_0>(x, x_bf16, M, K, W, N, bias, act, y, s);
    case kQ4_K: return launch_ks<kQ4_K>(x, x_bf16, M, K, W, N, bias, act, y, s);
    case kQ6_K: return launch_ks<kQ6_K>(x, x_bf16, M, K, W, N, bias, act, y, s);
    case kIQ4_NL: return launch_ks<kIQ4_NL>(x, x_bf16, M, K, W, N, bias, act, y, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv_ks: ggml type %d is not implemented", type);
    }
}

int launch_gemv_ks_batch(int type, int count, const XsBatchItem *items, hipStream_t s) {
    if (count < 1 || count > kMaxBatchKs) return fail(GQ_ERR_INVALID, "gemv batch: %d problems (1..%d supported per launch)", count, kMaxBatchKs);
    switch (type) {
    case kQ4_0: return launch_ks_batch<kQ4_0>(count, items, s);
    case kQ8_0: return launch_ks_batch<kQ8_0>(count, items, s);
    case kQ4_K: return launch_ks_batch<kQ4_K>(count, items, s);
    case kQ6_K: return launch_ks_batch<kQ6_K>(count, items, s);
    case kIQ4_NL: return launch_ks_batch<kIQ4_NL>(count, items, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv batch: ggml type %d is not implemented", type);
    }
}

}  // namespace gq
