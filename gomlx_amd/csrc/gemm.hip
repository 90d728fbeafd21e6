// Batched / prefill quantised Dense on the gfx950 matrix cores:
//   Y[m,n] = act(sum_k X[m,k] * w[n,k] + b[n]),  X [M,K],  W GGML blocks [N, row_bytes].
//
// A workgroup of 8 wavefronts owns a 256 x 128 tile of Y (256 activation rows, 128 weight
// rows); each wavefront a 64 x 64 sub-tile = 2 x 2 v_mfma_f32_32x32x16 accumulators.  Per
// 128-wide K step the workgroup dequantises its 128 x 128 slab of W (exact fp32 values, then one
// rounding to the 16-bit MFMA operand type) and stages the 256 x 128 slab of X next to it in
// LDS.  Both operands are K-contiguous, which is exactly the A / B fragment shape the
// instruction wants (8 consecutive k per lane), so fragments are single 16-byte LDS reads from
// rows padded to 272 bytes (conflict-free).
//
// The global loads of step k+1 are issued right after the barrier that publishes step k and
// wait in registers through the 32 MFMAs per wavefront of step k.
//
//   bf16 activations -> bf16 MFMA (the prefill path);
//   fp32 activations -> rounded to fp16, fp16 MFMA (11-bit operands; generic batched path).
#include "blocks.hpp"
#include "common.hpp"

namespace gq {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 128, BK = 128;
constexpr int LDS_STRIDE = BK + 8;  // 16-bit elements per LDS row: 256 B of data + 16 B pad
constexpr int LDS_BYTES = (BM + BN) * LDS_STRIDE * 2;

template <bool BF16> struct Operand;
template <> struct Operand<true> {
    typedef bf16x8 vec8;
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        bf2 v;
        v.x = (__bf16)a;
        v.y = (__bf16)b;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Operand<false> {
    typedef f16x8 vec8;
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 v;
        v.x = (_Float16)a;
        v.y = (_Float16)b;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// ---- raw (still packed) share of one thread in the W slab: one 32-value run of one row ---------
// Thread (row = t / 4, blk = t % 4) owns weights k0 + 32 blk .. + 31 of its row.
template <int T> struct WRaw;

template <> struct WRaw<kQ8_0> {
    uint32_t d;
    u128_a2 q0, q1;
    __device__ __forceinline__ void load(const uint8_t *row, int64_t kblk) {
        const uint8_t *blk = row + kblk * 34;
        d = load_u16(blk);
        q0 = *reinterpret_cast<const u128_a2 *>(blk + 2);
        q1 = *reinterpret_cast<const u128_a2 *>(blk + 18);
    }
    // int8 q = (q ^ 0x80) - 128 with the xor-ed byte read as unsigned; fma(u, d, -128 d) = d * q
    // exactly (the product has at most 18 significant bits), i.e. the reference's f32(d) * f32(q).
    __device__ __forceinline__ void values(float *w) const {
        const float df = half_bits_to_float(d), off = -128.0f * df;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t a = (i < 4 ? q0.v[i] : q1.v[i - 4]) ^ 0x80808080u;
            w[4 * i + 0] = fmaf(ubyte0(a), df, off);
            w[4 * i + 1] = fmaf(ubyte1(a), df, off);
            w[4 * i + 2] = fmaf(ubyte2(a), df, off);
            w[4 * i + 3] = fmaf(ubyte3(a), df, off);
        }
    }
};

// Other formats: keep the position and decode through the exact 16-value helper at store time.
template <int T> struct WRaw {
    const uint8_t *row;
    int64_t i16;
    __device__ __forceinline__ void load(const uint8_t *r, int64_t kblk) {
        row = r;
        i16 = kblk * 2;
    }
    __device__ __forceinline__ void values(float *w) const {
        dequant16<T>(row, i16, w);
        dequant16<T>(row, i16 + 1, w + 16);
    }
};

// The 256 x 128 activation slab as 16-byte chunks, chunk-major over the 512 threads: chunk
// g = 512 j + t (j-th load of thread t) is chunk g % CPR of row g / CPR, so consecutive lanes read
// consecutive 16 bytes of one row (a wavefront covers 4 full rows = 8 cache lines per load
// instead of 64 lines with a row-per-lane assignment, which leaves the kernel bound by the
// texture addresser).
template <bool BF16> struct XRaw;
template <> struct XRaw<true> {
    static constexpr int CPR = 16, NCH = 8;  // chunks per row (8 bf16 each), chunks per thread
    uint4 v[NCH];
    __device__ __forceinline__ void load(const void *X, int bm, int M, int k0, int K, int tid) {
        const uint16_t *p = reinterpret_cast<const uint16_t *>(X);
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            const int g = 512 * j + tid, row = g / CPR, k = k0 + (g % CPR) * 8;
            v[j] = *reinterpret_cast<const uint4 *>(p + (int64_t)min(bm + row, M - 1) * K + (k < K ? k : 0));
        }
    }
    __device__ __forceinline__ void store(uint16_t *xs, int bm, int M, int k0, int K, int tid) const {
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            const int g = 512 * j + tid, row = g / CPR, c = g % CPR;
            const bool ok = bm + row < M && k0 + c * 8 < K;
            *reinterpret_cast<uint4 *>(xs + row * LDS_STRIDE + c * 8) = ok ? v[j] : make_uint4(0, 0, 0, 0);
        }
    }
};
template <> struct XRaw<false> {
    static constexpr int CPR = 32, NCH = 16;  // chunks per row (4 fp32 each), chunks per thread
    float4 v[NCH];
    __device__ __forceinline__ void load(const void *X, int bm, int M, int k0, int K, int tid) {
        const float *p = reinterpret_cast<const float *>(X);
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            const int g = 512 * j + tid, row = g / CPR, k = k0 + (g % CPR) * 4;
            v[j] = *reinterpret_cast<const float4 *>(p + (int64_t)min(bm + row, M - 1) * K + (k < K ? k : 0));
        }
    }
    __device__ __forceinline__ void store(uint16_t *xs, int bm, int M, int k0, int K, int tid) const {
#pragma unroll
        for (int j = 0; j < NCH; j++) {
            const int g = 512 * j + tid, row = g / CPR, c = g % CPR;
            const bool ok = bm + row < M && k0 + c * 4 < K;
            const uint2 h = make_uint2(Operand<false>::pack(v[j].x, v[j].y), Operand<false>::pack(v[j].z, v[j].w));
            *reinterpret_cast<uint2 *>(xs + row * LDS_STRIDE + c * 4) = ok ? h : make_uint2(0, 0);
        }
    }
};

// X must be 16-byte aligned; K % 32 == 0.  One LDS stage of BK = 128: the MFMA phase of a step
// (32 MFMAs per wavefront) is long enough to cover the global-memory latency of the next
// step's loads, which wait in registers and are converted and stored between two barriers.
template <int T, bool BF16>
__global__ __launch_bounds__(512) void gemm_kernel(const void *__restrict__ Xv, const uint8_t *__restrict__ W,
                                                   const float *__restrict__ bias, float *__restrict__ Y, int M, int K,
                                                   int N, int64_t row_bytes, int act) {
    typedef Operand<BF16> Op;
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];

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

    // staging role for W: 128 rows x 4 runs of 32 weights
    const int wrow_i = tid >> 2, wblk = tid & 3;
    const uint8_t *wrow = W + (int64_t)min(bn + wrow_i, N - 1) * row_bytes;
    uint16_t *wdst = lds + (BM + wrow_i) * LDS_STRIDE + 32 * wblk;

    XRaw<BF16> xr[1];
    WRaw<T> wr[1];
    const int nk = (K + BK - 1) / BK;
    const int64_t nblk32 = K >> 5;
    auto fetch = [&](int kt, XRaw<BF16> &x, WRaw<T> &w) {
        const int k0 = kt * BK;
        x.load(Xv, bm, M, k0, K, tid);
        w.load(wrow, min((int64_t)(k0 >> 5) + wblk, nblk32 - 1));
    };
    auto stage = [&](int kt, const XRaw<BF16> &x, const WRaw<T> &wq) {
        const int k0 = kt * BK;
        x.store(lds, bm, M, k0, K, tid);
        float w[32];
        wq.values(w);
        const bool w_ok = k0 + 32 * wblk < K;
        uint4 *d = reinterpret_cast<uint4 *>(wdst);
#pragma unroll
        for (int j = 0; j < 4; j++)
            d[j] = w_ok ? make_uint4(Op::pack(w[8 * j], w[8 * j + 1]), Op::pack(w[8 * j + 2], w[8 * j + 3]),
                                     Op::pack(w[8 * j + 4], w[8 * j + 5]), Op::pack(w[8 * j + 6], w[8 * j + 7]))
                        : make_uint4(0, 0, 0, 0);
    };
    const uint16_t *xs = lds, *ws = lds + BM * LDS_STRIDE;
    auto contract = [&]() {
#pragma unroll
        for (int kk = 0; kk < BK / 16; kk++) {
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
    };

    fetch(0, xr[0], wr[0]);
    for (int kt = 0; kt < nk; kt++) {
        stage(kt, xr[0], wr[0]);
        __syncthreads();
        fetch(min(kt + 1, nk - 1), xr[0], wr[0]);  // unconditional (clamped): in flight during the MFMA phase
        contract();
        __syncthreads();
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
    static const bool lds_ok = [] {
        return hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_kernel<T, BF16>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) == hipSuccess;
    }();
    if (!lds_ok) return fail(GQ_ERR_HIP, "gemm: cannot reserve %d bytes of LDS", LDS_BYTES);
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    const dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
    return launch(gemm_kernel<T, BF16>, grid, dim3(512), (size_t)LDS_BYTES, s, x, W, bias, y, (int)M, (int)K, (int)N, row_bytes,
                  act);
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
    if (reinterpret_cast<uintptr_t>(x) & 15)
        return fail(GQ_ERR_NOT_IMPLEMENTED, "qdense: batched activations that are not 16-byte aligned are not implemented");
    switch (type) {
    case kQ4_0: return launch_type<kQ4_0>(x_is_bf16, x, M, K, W, N, bias, act, y, s);
    case kQ8_0: return launch_type<kQ8_0>(x_is_bf16, x, M, K, W, N, bias, act, y, s);
    case kIQ4_NL: return launch_type<kIQ4_NL>(x_is_bf16, x, M, K, W, N, bias, act, y, s);
    case kQ4_K: return launch_type<kQ4_K>(x_is_bf16, x, M, K, W, N, bias, act, y, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "qdense: ggml type %d is not implemented", type);
    }
}

}  // namespace gq
