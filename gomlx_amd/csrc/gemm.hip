// Batched / prefill quantised Dense on the gfx950 matrix cores:
//   Y[m,n] = act(sum_k X[m,k] * w[n,k] + b[n]),  X [M,K],  W GGML blocks [N, row_bytes].
//
// Each workgroup owns a BM x BN tile of Y.  Per 32-wide K step it dequantises its BN x 32
// slab of W (exact fp32 values, then rounded once to the 16-bit MFMA operand type) into
// LDS, stages the BM x 32 slab of X beside it, and the wavefronts contract the two slabs
// with v_mfma_f32_32x32x16 (fp32 accumulation).  Both operands are K-contiguous, which is
// exactly the A / B fragment shape the instruction wants (8 consecutive k per lane).
//
//   bf16 activations -> bf16 MFMA (the prefill path);
//   fp32 activations -> rounded to fp16, fp16 MFMA (11-bit operands, small-batch path).
#include "blocks.hpp"
#include "common.hpp"

namespace gq {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int LDS_STRIDE = 40;  // 16-bit elements per LDS row: 64 B of data + 16 B pad (conflict-free ds_read_b128)

template <bool BF16> struct Operand;
template <> struct Operand<true> {
    typedef bf16x8 vec8;
    static __device__ __forceinline__ uint16_t from_float(float f) {
        const __bf16 b = (__bf16)f;
        return __builtin_bit_cast(uint16_t, b);
    }
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Operand<false> {
    typedef f16x8 vec8;
    static __device__ __forceinline__ uint16_t from_float(float f) {
        const _Float16 h = (_Float16)f;
        return __builtin_bit_cast(uint16_t, h);
    }
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

__device__ __forceinline__ uint32_t pack2(uint16_t lo, uint16_t hi) { return (uint32_t)lo | ((uint32_t)hi << 16); }

template <int T, bool BF16>
__global__ __launch_bounds__(256) void gemm_kernel(const void *__restrict__ Xv, const uint8_t *__restrict__ W,
                                                   const float *__restrict__ bias, float *__restrict__ Y, int M, int K,
                                                   int N, int64_t row_bytes, int act) {
    typedef Operand<BF16> Op;
    __shared__ __attribute__((aligned(16))) uint16_t xs[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t ws[BN * LDS_STRIDE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bm = blockIdx.y * BM, bn = blockIdx.x * BN;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // staging role of this thread: row (tid / 2) of the slab, 16-element half (tid % 2)
    const int srow = tid >> 1, shalf = tid & 1;
    const int xm = bm + srow, wn_row = bn + srow;
    const uint8_t *wrow = W + (int64_t)min(wn_row, N - 1) * row_bytes;

    for (int k0 = 0; k0 < K; k0 += BK) {
        // ---- X slab -> LDS
        uint32_t xp[8];
        if (xm < M) {
            if constexpr (BF16) {
                const uint16_t *xr = reinterpret_cast<const uint16_t *>(Xv) + (int64_t)xm * K + k0 + 16 * shalf;
#pragma unroll
                for (int j = 0; j < 8; j++) xp[j] = pack2(xr[2 * j], xr[2 * j + 1]);
            } else {
                const float *xr = reinterpret_cast<const float *>(Xv) + (int64_t)xm * K + k0 + 16 * shalf;
#pragma unroll
                for (int j = 0; j < 8; j++) xp[j] = pack2(Op::from_float(xr[2 * j]), Op::from_float(xr[2 * j + 1]));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) xp[j] = 0u;
        }
        // ---- W slab: exact fp32 dequantisation, one rounding to the operand type
        float wv[16];
        dequant16<T>(wrow, (int64_t)(k0 >> 4) + shalf, wv);
        uint32_t wp[8];
#pragma unroll
        for (int j = 0; j < 8; j++) wp[j] = pack2(Op::from_float(wv[2 * j]), Op::from_float(wv[2 * j + 1]));

        if (k0 > 0) __syncthreads();
        uint4 *xd = reinterpret_cast<uint4 *>(&xs[srow * LDS_STRIDE + 16 * shalf]);
        xd[0] = make_uint4(xp[0], xp[1], xp[2], xp[3]);
        xd[1] = make_uint4(xp[4], xp[5], xp[6], xp[7]);
        uint4 *wd = reinterpret_cast<uint4 *>(&ws[srow * LDS_STRIDE + 16 * shalf]);
        wd[0] = make_uint4(wp[0], wp[1], wp[2], wp[3]);
        wd[1] = make_uint4(wp[4], wp[5], wp[6], wp[7]);
        __syncthreads();

        // ---- contract: two K=16 MFMA steps over the 32-wide slab
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const int koff = kk * 16 + (lane >> 5) * 8;
            typename Op::vec8 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; i++)
                a[i] = *reinterpret_cast<const typename Op::vec8 *>(&xs[(wm + i * 32 + (lane & 31)) * LDS_STRIDE + koff]);
#pragma unroll
            for (int j = 0; j < 2; j++)
                b[j] = *reinterpret_cast<const typename Op::vec8 *>(&ws[(wn + j * 32 + (lane & 31)) * LDS_STRIDE + koff]);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = Op::mfma(a[i], b[j], acc[i][j]);
        }
    }

    // ---- epilogue: acc[i][j][r] is Y[m, n] with n = lane % 32, m = 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int n = bn + wn + j * 32 + (lane & 31);
        if (n >= N) continue;
        const float bv = bias ? bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = bm + wm + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < M) Y[(int64_t)m * N + n] = apply_act(act, acc[i][j][r] + bv);
            }
        }
    }
}

template <int T, bool BF16>
int launch_one(const void *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
               hipStream_t s) {
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    const dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
    return launch(gemm_kernel<T, BF16>, grid, dim3(256), 0, s, x, W, bias, y, (int)M, (int)K, (int)N, row_bytes, act);
}

template <int T>
int launch_type(bool bf16, const void *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act,
                float *y, hipStream_t s) {
    return bf16 ? launch_one<T, true>(x, M, K, W, N, bias, act, y, s)
                : launch_one<T, false>(x, M, K, W, N, bias, act, y, s);
}

}  // namespace

int launch_gemm(int type, bool x_is_bf16, const void *x, int64_t M, int64_t K, const uint8_t *W, int64_t N,
                const float *bias, int act, float *y, hipStream_t s) {
    if (M == 0 || N == 0) return GQ_OK;
    if (N > INT32_MAX || K > INT32_MAX || M > INT32_MAX || (M + BM - 1) / BM > 65535)
        return fail(GQ_ERR_NOT_IMPLEMENTED, "gemm: dimensions M=%lld K=%lld N=%lld exceed the kernel's index range",
                    (long long)M, (long long)K, (long long)N);
    switch (type) {
    case kQ4_0: return launch_type<kQ4_0>(x_is_bf16, x, M, K, W, N, bias, act, y, s);
    case kQ8_0: return launch_type<kQ8_0>(x_is_bf16, x, M, K, W, N, bias, act, y, s);
    case kIQ4_NL: return launch_type<kIQ4_NL>(x_is_bf16, x, M, K, W, N, bias, act, y, s);
    case kQ4_K: return launch_type<kQ4_K>(x_is_bf16, x, M, K, W, N, bias, act, y, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "qdense: ggml type %d is not implemented", type);
    }
}

}  // namespace gq
