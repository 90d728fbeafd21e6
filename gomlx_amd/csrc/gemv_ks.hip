// Decode GEMV, K-sliced integer-dot kernels (Q4_0, Q8_0, Q4_K, Q6_K, IQ4_NL; K % 256 == 0): the
// kernels and launchers of the plain dense call and of batched submission.  The work of a
// workgroup is in gemv_ks_body.hpp.
#include "gemv_ks_body.hpp"

namespace gq {

namespace {

// grid.y passes of R activation rows each (the last one may hold fewer)
template <int T, int PF, int WIN, bool XBF16, int R>
__global__ __launch_bounds__(512) void gemv_ks_kernel(const void *__restrict__ X, const uint8_t *__restrict__ W,
                                                      const float *__restrict__ bias, float *__restrict__ Y, int M, int K, int N,
                                                      int64_t row_bytes, int iters, int nslices, int half_tail, int act) {
    extern __shared__ uint32_t lds[];
    const int64_t x_stride = (int64_t)K * (XBF16 ? 2 : 4);
    const int r0 = (int)blockIdx.y * R;
    const uint8_t *x = reinterpret_cast<const uint8_t *>(X) + r0 * x_stride;
    ks_body<T, PF, WIN, false, XBF16, R>(x, W, bias, Y + (int64_t)r0 * N, N, row_bytes, iters, nslices, half_tail, act, (int)(blockDim.x >> 6),
                                         (int)blockIdx.x, lds, nullptr, min(R, M - r0), x_stride, 0, (int)gridDim.x);
}

template <int T>
__global__ __launch_bounds__(512) void gemv_ks_batch_kernel(const KsBatch b) {
    extern __shared__ uint32_t lds[];
    const KsProblem &q = b.p[ks_batch_problem(b, (int)blockIdx.x)];
    const int64_t row = blockIdx.y;  // activation row of every problem
    ks_body<T, kBatchPF, kBatchWin, false, false, 1, true>(q.x + row * q.K, q.W, q.bias, q.y + row * q.N, q.N, q.row_bytes, q.iters, q.nslices, q.half_tail, q.act, q.waves,
                     (int)blockIdx.x - q.wg_begin, lds, nullptr, 1, 0, q.live, q.nwg);
}


template <int T, int PF, int R = 1>
int launch_ks_pf(const KsPlan &p, const void *x, int x_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act,
                 float *y, hipStream_t s) {
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    const dim3 grid((unsigned)p.wgs, (unsigned)((M + R - 1) / R)), block((unsigned)p.waves * 64);
    constexpr int WIN = PF < 3 ? PF : 3;
    const size_t shmem = ks_lds_bytes(p.waves, p.iters, R);
    if (x_bf16)
        return launch(gemv_ks_kernel<T, PF, WIN, true, R>, grid, block, shmem, s, x, W, bias, y, (int)M, (int)K, (int)N, row_bytes, p.iters,
                      p.nslices, p.half_tail, act);
    return launch(gemv_ks_kernel<T, PF, WIN, false, R>, grid, block, shmem, s, x, W, bias, y, (int)M, (int)K, (int)N, row_bytes, p.iters,
                  p.nslices, p.half_tail, act);
}

// Batches: passes of two rows for two, of four rows for more (groups of 1, 2 or 4 row-steps only, to
// keep the number of kernel variants down).
template <int T, int R>
int launch_ks_rows(KsPlan p, const void *x, int x_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act,
                   float *y, hipStream_t s) {
    ks_regroup(p, N, false, R == 4 ? 2 : 4);
    switch (p.pf) {
    case 1: return launch_ks_pf<T, 1, R>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    case 2: return launch_ks_pf<T, 2, R>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    default:
        if constexpr (R == 4) return fail(GQ_ERR_HIP, "gemv_ks: no such kernel");
        else return launch_ks_pf<T, 4, R>(p, x, x_bf16, M, K, W, N, bias, act, y, s);
    }
}

template <int T>
int launch_ks(const void *x, int x_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
              hipStream_t s) {
    KsPlan p;
    if (!ks_plan(K, N, p)) return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv_ks: unsupported problem");
    // Batches over a large matrix: passes of up to four rows against one reading of W (a pass per row re-reads it:
    // Q8_0 4096 -> 14336 at 4 rows 35.4 us, one pass of four 15.8 us).  Small matrices stay in cache between the
    // concurrent passes of single rows, which then cost less than the arithmetic of a multi-row pass
    // (Q4_0 4096 x 4096 at 4 rows: 9.4 us as four passes, 10.7 us as one).
    if (M > 1 && (int64_t)gq_row_bytes(T, K) * N >= kLargeWeightBytes) {
        constexpr int RM = ks_max_rows<T>();
        const int64_t full = M / RM * RM, rem = M - full;
        const int64_t xb = K * (x_bf16 ? 2 : 4);
        if (full)
            if (int rc = launch_ks_rows<T, RM>(p, x, x_bf16, full, K, W, N, bias, act, y, s)) return rc;
        const void *xr = static_cast<const uint8_t *>(x) + full * xb;
        float *yr = y + full * N;
        if (rem == 2 || (rem == 3 && RM < 4)) {
            if (int rc = launch_ks_rows<T, 2>(p, xr, x_bf16, rem, K, W, N, bias, act, yr, s)) return rc;
            return GQ_OK;
        }
        if (rem == 3) return launch_ks_rows<T, RM>(p, xr, x_bf16, rem, K, W, N, bias, act, yr, s);
        if (rem == 0) return GQ_OK;
        x = xr;  // one row left: the single-row kernel below
        y = yr;
        M = 1;
    }
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
int launch_ks_batch(int count, const XsBatchItem *items, int rows, hipStream_t s) {
    KsBatch b;
    size_t shmem;
    int wgs;
    if (int rc = plan_ks_batch<T>(count, items, b, shmem, wgs)) return rc;
    return launch(gemv_ks_batch_kernel<T>, dim3((unsigned)wgs, (unsigned)rows), dim3(512), shmem, s, b);
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

int launch_gemv_ks_batch(int type, int count, const XsBatchItem *items, hipStream_t s, int rows) {
    if (count < 1 || count > kMaxBatchKs) return fail(GQ_ERR_INVALID, "gemv batch: %d problems (1..%d supported per launch)", count, kMaxBatchKs);
    switch (type) {
    case kQ4_0: return launch_ks_batch<kQ4_0>(count, items, rows, s);
    case kQ8_0: return launch_ks_batch<kQ8_0>(count, items, rows, s);
    case kQ4_K: return launch_ks_batch<kQ4_K>(count, items, rows, s);
    case kQ6_K: return launch_ks_batch<kQ6_K>(count, items, rows, s);
    case kIQ4_NL: return launch_ks_batch<kIQ4_NL>(count, items, rows, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv batch: ggml type %d is not implemented", type);
    }
}

}  // namespace gq
