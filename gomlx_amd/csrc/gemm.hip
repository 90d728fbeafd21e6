// Batched / prefill quantised Dense on the gfx950 matrix cores:
//   Y[m,n] = act(sum_k X[m,k] * w[n,k] + b[n]),  X [M,K],  W GGML blocks [N, row_bytes].
//
// A workgroup of 8 wavefronts owns a 256 x 128 tile of Y (256 activation rows, 128 weight
// rows); each wavefront a 64 x 64 sub-tile = 2 x 2 v_mfma_f32_32x32x16 accumulators.  K advances
// in steps of 64 through two LDS buffers: while the matrix cores contract step k out of one
// buffer, the same wavefronts dequantise the 128 x 64 slab of W of step k+1 (exact fp32 values,
// then one rounding to the 16-bit MFMA operand type) and copy the 256 x 64 slab of X into the
// other buffer, so the vector ALU work hides in the shadow of the MFMAs and one barrier per step
// suffices.  The global loads run two steps ahead of the staging, in two register sets.
// Both operands are K-contiguous, which is exactly the A / B fragment shape the instruction
// wants (8 consecutive k per lane), so fragments are single 16-byte LDS reads from rows padded
// to 144 bytes (conflict-free).
//
//   bf16 activations -> bf16 MFMA (the prefill path);
//   fp32 activations -> rounded to fp16, fp16 MFMA (11-bit operands; generic batched path).
#include "blocks.hpp"
#include "common.hpp"

#include <type_traits>

namespace gq {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 128, BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // 16-bit elements per LDS row: 128 B of data + 16 B pad
constexpr int LDS_BUF = (BM + BN) * LDS_STRIDE;  // elements per buffer
constexpr int LDS_BYTES = 2 * LDS_BUF * 2;

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

// ---- raw (still packed) share of one thread in the W slab: one 16-value run of one row ---------
// Thread (row = t / 4, run = t % 4) owns weights k0 + 16 run .. + 15 of its row.
template <int T> struct WRaw;

template <> struct WRaw<kQ8_0> {
    uint32_t d;
    u128_a2 q;
    // `base` is uniform (first row of the tile, block column of the K step); `off` is this thread's
    // constant byte offset of its block within the tile.
    __device__ __forceinline__ void set_row(const uint8_t *) {}
    __device__ __forceinline__ void load(const uint8_t *base, uint32_t off, uint32_t run, int64_t) {
        const uint8_t *blk = base + off;
        d = load_u16(blk);
        q = *reinterpret_cast<const u128_a2 *>(blk + 2 + 16 * (run & 1));
    }
    // Values 4 part .. 4 part + 3 of the run: f32(d) * f32(q), the reference's product (exact: at most 18 significant
    // bits), each int8 converted by one instruction.
    __device__ __forceinline__ void part(int i, float *w) const {
        const float df = half_bits_to_float(d);
        const uint32_t a = q.v[i];
        w[4 * i + 0] = sbyte0(a) * df;
        w[4 * i + 1] = sbyte1(a) * df;
        w[4 * i + 2] = sbyte2(a) * df;
        w[4 * i + 3] = sbyte3(a) * df;
    }
};

// Other formats: keep the position and decode through the exact 16-value helper at store time.
template <int T> struct WRaw {
    const uint8_t *row;
    int64_t i16;
    __device__ __forceinline__ void set_row(const uint8_t *r) { row = r; }
    __device__ __forceinline__ void load(const uint8_t *, uint32_t, uint32_t, int64_t i) { i16 = i; }
    __device__ __forceinline__ void part(int i, float *w) const {
        if (i == 0) dequant16<T>(row, i16, w);
    }
};

// The 256 x 64 activation slab as 16-byte chunks, chunk-major over the 512 threads: chunk
// g = 512 j + t (j-th load of thread t) is chunk g % CPR of row g / CPR, so consecutive lanes read
// consecutive 16 bytes of one row (a row-per-lane assignment touches 64 cache lines per load
// and leaves the kernel bound by the texture addresser).
template <bool BF16> struct XRaw;
__device__ __forceinline__ uint32_t all_ones_if(bool c) { return c ? 0xFFFFFFFFu : 0u; }
// Addressing: a uniform base pointer (tile row 0, column of the K step) advances on the scalar unit;
// each thread adds constant 32-bit byte offsets (its row, clamped to M - 1, and its chunk).  In a
// last step that covers only 32 columns the chunks of the missing half re-read the first half;
// store_part zeroes them.
template <> struct XRaw<true> {
    static constexpr int CPR = 8, NCH = 4;  // chunks per row (8 bf16 each), chunks per thread
    static constexpr int ESIZE = 2;
    uint4 v[NCH];
    static __device__ __forceinline__ uint32_t offset(int j, int bm, int M, int K, int tid, bool tail) {
        const int g = 512 * j + tid, row = g / CPR;
        int c = g % CPR;
        if (tail && c >= CPR / 2) c -= CPR / 2;
        return (uint32_t)(min(row, M - 1 - bm) * K + c * 8) * ESIZE;
    }
    __device__ __forceinline__ void load(const uint8_t *base, const uint32_t *off) {
#pragma unroll
        for (int j = 0; j < NCH; j++) v[j] = *reinterpret_cast<const uint4 *>(base + off[j]);
    }
    // the loads that refill what store_part(i) has just consumed
    __device__ __forceinline__ void load_part(int i, const uint8_t *base, const uint32_t *off) {
        v[i] = *reinterpret_cast<const uint4 *>(base + off[i]);
    }
    // Part i of 4 of the copy into LDS.  Columns at or beyond K become zero; rows beyond M hold a
    // copy of row M - 1 and only feed outputs that are never written.
    // MASKED = false is for steps that lie entirely inside K.
    template <bool MASKED>
    __device__ __forceinline__ void store_part(int i, uint16_t *xs, int k0, int K, int tid) const {
        const int g = 512 * i + tid, row = g / CPR, c = g % CPR;
        const uint32_t m = MASKED ? all_ones_if(k0 + c * 8 < K) : 0xFFFFFFFFu;
        *reinterpret_cast<uint4 *>(xs + row * LDS_STRIDE + c * 8) = make_uint4(v[i].x & m, v[i].y & m, v[i].z & m, v[i].w & m);
    }
};
template <> struct XRaw<false> {
    static constexpr int CPR = 16, NCH = 8;  // chunks per row (4 fp32 each), chunks per thread
    static constexpr int ESIZE = 4;
    float4 v[NCH];
    static __device__ __forceinline__ uint32_t offset(int j, int bm, int M, int K, int tid, bool tail) {
        const int g = 512 * j + tid, row = g / CPR;
        int c = g % CPR;
        if (tail && c >= CPR / 2) c -= CPR / 2;
        return (uint32_t)(min(row, M - 1 - bm) * K + c * 4) * ESIZE;
    }
    __device__ __forceinline__ void load(const uint8_t *base, const uint32_t *off) {
#pragma unroll
        for (int j = 0; j < NCH; j++) v[j] = *reinterpret_cast<const float4 *>(base + off[j]);
    }
    __device__ __forceinline__ void load_part(int i, const uint8_t *base, const uint32_t *off) {
        v[2 * i] = *reinterpret_cast<const float4 *>(base + off[2 * i]);
        v[2 * i + 1] = *reinterpret_cast<const float4 *>(base + off[2 * i + 1]);
    }
    template <bool MASKED>
    __device__ __forceinline__ void store_part(int i, uint16_t *xs, int k0, int K, int tid) const {
#pragma unroll
        for (int j = 2 * i; j < 2 * i + 2; j++) {
            const int g = 512 * j + tid, row = g / CPR, c = g % CPR;
            const uint32_t m = MASKED ? all_ones_if(k0 + c * 4 < K) : 0xFFFFFFFFu;
            *reinterpret_cast<uint2 *>(xs + row * LDS_STRIDE + c * 4) =
                make_uint2(Operand<false>::pack(v[j].x, v[j].y) & m, Operand<false>::pack(v[j].z, v[j].w) & m);
        }
    }
};


// X must be 16-byte aligned; K % 32 == 0.
// KTAIL: K is not a multiple of the 64-wide step (the last step covers 32 columns); without it the step's address
// selects and masks drop out of the loop.
template <int T, bool BF16, bool KTAIL>
// (Xv and W are deliberately not __restrict__: loads through restrict-qualified read-only pointers
// may be moved across the workgroup barriers, away from the place that gives them two steps of
// latency cover.)
__global__ __launch_bounds__(512) void gemm_kernel(const void *Xv, const uint8_t *W,
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

    // staging role for W: 128 rows x 4 runs of 16 weights
    const int wrow_i = tid >> 2, wrun = tid & 3;
    const int wrow_c = min(wrow_i, N - 1 - bn);  // clamped row within the tile
    const int wdst_off = (BM + wrow_i) * LDS_STRIDE + 16 * wrun;

    XRaw<BF16> xr[2];
    WRaw<T> wr[2];
    wr[0].set_row(W + (int64_t)(bn + wrow_c) * row_bytes);
    wr[1].set_row(W + (int64_t)(bn + wrow_c) * row_bytes);
    const int nk = (K + BK - 1) / BK;
    const int64_t n16 = K >> 4;
    constexpr bool ktail = KTAIL;  // the last step covers 32 columns only
    // constant per-thread byte offsets, for full steps and for a half last step
    uint32_t xoff[XRaw<BF16>::NCH], xoff_t[XRaw<BF16>::NCH];
#pragma unroll
    for (int j = 0; j < XRaw<BF16>::NCH; j++) {
        xoff[j] = XRaw<BF16>::offset(j, bm, M, K, tid, false);
        xoff_t[j] = XRaw<BF16>::offset(j, bm, M, K, tid, true);
    }
    const uint32_t woff = (uint32_t)(wrow_c * row_bytes) + (uint32_t)(wrun >> 1) * 34u;
    const uint32_t woff_t = (uint32_t)(wrow_c * row_bytes);  // half last step: runs 2, 3 re-read block 0
    const uint8_t *xtile = reinterpret_cast<const uint8_t *>(Xv) + (int64_t)bm * K * XRaw<BF16>::ESIZE;
    const uint8_t *wtile = W + (int64_t)bn * row_bytes;
    auto fetch = [&](int kt, XRaw<BF16> &x, WRaw<T> &w) __attribute__((always_inline)) {  // unconditional: steps past the end re-read the last one
        const int kc = min(kt, nk - 1);  // uniform
        const bool tail = ktail && kc == nk - 1;
        const uint8_t *xb = xtile + (int64_t)kc * (BK * XRaw<BF16>::ESIZE);
        uint32_t o[XRaw<BF16>::NCH];
#pragma unroll
        for (int j = 0; j < XRaw<BF16>::NCH; j++) o[j] = tail ? xoff_t[j] : xoff[j];
        x.load(xb, o);
        w.load(wtile + (int64_t)kc * (BK / 32 * 34), tail ? woff_t : woff, (uint32_t)wrun,
               min((int64_t)kc * (BK / 16) + wrun, n16 - 1));
    };
    // One K step.  The MFMAs run in four groups of four, each group followed in program order by a
    // quarter of the staging of step kt + 1 into `nxt` (MFMAs are issued asynchronously, so the
    // vector ALU work that follows them runs in their shadow).  Fragments are read one group ahead,
    // and the groups are skewed by one against the barriers: a step opens with the reads of its
    // own group 0 and the MFMAs of the previous step's group 3, whose fragments were read before
    // the barrier, so the matrix cores have work while the first LDS reads after a barrier are in
    // flight.  The scheduling barriers keep the compiler from regrouping this.
    // (The fp32-activation variants hold twice the activation registers and keep the plain order:
    // carrying fragments across the barrier pushes some of them over the register budget.)
    constexpr bool SKEW = BF16;
    typename Op::vec8 fa[2][2], fb[2][2];  // [set][tile]; with SKEW set 1 carries group 3 across the barrier
    auto mfma_group = [&](int set) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) acc[i][j] = Op::mfma(fa[set][i], fb[set][j], acc[i][j]);
    };
    auto step = [&](int kt, const uint16_t *cur, uint16_t *nxt, XRaw<BF16> &x, WRaw<T> &wq, auto masked, auto first) __attribute__((always_inline)) {
        constexpr bool MASKED = decltype(masked)::value, FIRST = decltype(first)::value;
        const uint16_t *xs = cur, *ws = cur + BM * LDS_STRIDE;
        const int k1 = (kt + 1) * BK;
        // the register set staged here is refilled, piece by piece, with step kt + 3
        const int kc = min(kt + 3, nk - 1);  // uniform; steps past the end re-read the last one
        const bool ftail = ktail && kc == nk - 1;
        const uint8_t *xb = xtile + (int64_t)kc * (BK * XRaw<BF16>::ESIZE);
        uint32_t fo[XRaw<BF16>::NCH];
#pragma unroll
        for (int j = 0; j < XRaw<BF16>::NCH; j++) fo[j] = ftail ? xoff_t[j] : xoff[j];
        const uint32_t wmask = MASKED ? all_ones_if(k1 + 16 * wrun < K) : 0xFFFFFFFFu;
        uint4 *wd = reinterpret_cast<uint4 *>(nxt + wdst_off);
        auto frags = [&](int kk) __attribute__((always_inline)) {
            const int koff = kk * 16 + (lane >> 5) * 8, set = kk & 1;
#pragma unroll
            for (int i = 0; i < 2; i++)
                fa[set][i] = *reinterpret_cast<const typename Op::vec8 *>(&xs[(wm + i * 32 + (lane & 31)) * LDS_STRIDE + koff]);
#pragma unroll
            for (int j = 0; j < 2; j++)
                fb[set][j] = *reinterpret_cast<const typename Op::vec8 *>(&ws[(wn + j * 32 + (lane & 31)) * LDS_STRIDE + koff]);
        };
        float w[16];
        if (!SKEW) frags(0);
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            if (SKEW) {
                frags(kk);
                if (kk > 0 || !FIRST) mfma_group((kk + 1) & 1);  // group kk - 1 (kk = 0: group 3 of the step before)
            } else {
                if (kk < 3) frags(kk + 1);
                mfma_group(kk & 1);
            }
            x.template store_part<MASKED>(kk, nxt, k1, K, tid);
            wq.part(kk, w);
            x.load_part(kk, xb, fo);
            if (kk == 1 || kk == 3) {
                const int o = (kk >> 1) * 8;
                wd[kk >> 1] = make_uint4(Op::pack(w[o], w[o + 1]) & wmask, Op::pack(w[o + 2], w[o + 3]) & wmask,
                                         Op::pack(w[o + 4], w[o + 5]) & wmask, Op::pack(w[o + 6], w[o + 7]) & wmask);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        wq.load(wtile + (int64_t)kc * (BK / 32 * 34), ftail ? woff_t : woff, (uint32_t)wrun,
                min((int64_t)kc * (BK / 16) + wrun, n16 - 1));
    };
    auto stage_first = [&](uint16_t *buf, const XRaw<BF16> &x, const WRaw<T> &wq) __attribute__((always_inline)) {
        float w[16];
        const uint32_t wmask = all_ones_if(16 * wrun < K);
        uint4 *wd = reinterpret_cast<uint4 *>(buf + wdst_off);
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            x.template store_part<true>(kk, buf, 0, K, tid);
            wq.part(kk, w);
        }
#pragma unroll
        for (int h = 0; h < 2; h++)
            wd[h] = make_uint4(Op::pack(w[8 * h], w[8 * h + 1]) & wmask, Op::pack(w[8 * h + 2], w[8 * h + 3]) & wmask,
                               Op::pack(w[8 * h + 4], w[8 * h + 5]) & wmask, Op::pack(w[8 * h + 6], w[8 * h + 7]) & wmask);
    };

    // Step s is staged (registers -> LDS buffer s % 2) during step s - 1 out of register set s % 2,
    // which was filled by fetch(s) during step s - 3.  Steps come in pairs so that every pass of
    // the loop body issues the same loads (the wait counters then stay exact); a step past the end
    // of K stages zeros.
    // (the scheduling barriers pin the order of issue, which is what the wait counts in the loop
    // are derived from)
    fetch(0, xr[0], wr[0]);
    __builtin_amdgcn_sched_barrier(0);
    fetch(1, xr[1], wr[1]);
    __builtin_amdgcn_sched_barrier(0);
    stage_first(lds, xr[0], wr[0]);
    __builtin_amdgcn_sched_barrier(0);
    fetch(2, xr[0], wr[0]);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    auto pair = [&](int kt, auto masked, auto first) __attribute__((always_inline)) {
        step(kt, lds, lds + LDS_BUF, xr[1], wr[1], masked, first);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        step(kt + 1, lds + LDS_BUF, lds, xr[0], wr[0], masked, std::false_type());
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    };
    // The first pair runs outside the loop so that the loop is entered with exactly the loads in
    // flight that its own back edge leaves (otherwise the wait counts at the loop head are derived
    // from the prologue's different order and over-wait).  Pairs whose staged steps (kt + 1, kt + 2)
    // lie entirely inside K skip the zero-fill masks.
    const int nk_full = K / BK;
    pair(0, std::true_type(), std::true_type());
    int kt = 2;
    for (; kt + 2 < nk_full; kt += 2) pair(kt, std::false_type(), std::false_type());
    for (; kt < nk; kt += 2) pair(kt, std::true_type(), std::false_type());
    if (SKEW) mfma_group(1);  // group 3 of the last step

    // ---- epilogue: acc[i][j][r] is Y[m, n] with n = lane % 32, m = 8*(r/4) + 4*(lane/32) + r%4
    // Per element: one add, the activation, one store; the address is a per-lane base plus an offset that is the same for
    // the whole wavefront, and what does not depend on the element - which activation, whether the tile reaches over the
    // edge of the matrix - is decided once, outside the 64 stores.  (Written as one loop with those tests inside, the
    // compiler spent some twenty vector-ALU instructions per element: C3 took 84.4 us against 79.3.)
    const int m0 = bm + wm + 4 * (lane >> 5);
    auto store_all = [&](auto bounded, auto activate) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int n = bn + wn + j * 32 + (lane & 31);
            if constexpr (decltype(bounded)::value) { if (n >= N) continue; }
            const float bv = bias ? bias[n] : 0.f;
            float *__restrict__ yp = Y + (int64_t)m0 * N + n;
#pragma unroll
            for (int i = 0; i < 2; i++) {
                // a block of 32 rows is inside the matrix as a whole, outside as a whole, or (one block per tile column at most) cut by its edge
                const int rows_left = decltype(bounded)::value ? M - (bm + wm + i * 32) : 32;
                if (rows_left <= 0) continue;
                auto store16 = [&](auto checked) __attribute__((always_inline)) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int dm = i * 32 + 8 * (r >> 2) + (r & 3);
                        if constexpr (decltype(checked)::value) { if (m0 + dm >= M) continue; }
                        yp[(int64_t)dm * N] = activate(acc[i][j][r] + bv);
                    }
                };
                if (rows_left >= 32) store16(std::false_type());
                else store16(std::true_type());
            }
        }
    };
    auto by_act = [&](auto bounded) __attribute__((always_inline)) {
        if (act == kActNone) store_all(bounded, [](float v) { return v; });
        else store_all(bounded, [act](float v) { return apply_act(act, v); });
    };
    if (bm + BM <= M && bn + BN <= N) by_act(std::false_type());
    else by_act(std::true_type());
}

template <int T, bool BF16, bool KTAIL>
int launch_one_k(const void *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
               hipStream_t s) {
    static const bool lds_ok = [] {
        return hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_kernel<T, BF16, KTAIL>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) == hipSuccess;
    }();
    if (!lds_ok) return fail(GQ_ERR_HIP, "gemm: cannot reserve %d bytes of LDS", LDS_BYTES);
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    const dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
    return launch(gemm_kernel<T, BF16, KTAIL>, grid, dim3(512), (size_t)LDS_BYTES, s, x, W, bias, y, (int)M, (int)K, (int)N, row_bytes,
                  act);
}

template <int T, bool BF16>
int launch_one(const void *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y, hipStream_t s) {
    return K % BK ? launch_one_k<T, BF16, true>(x, M, K, W, N, bias, act, y, s) : launch_one_k<T, BF16, false>(x, M, K, W, N, bias, act, y, s);
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
    case kQ6_K: return launch_type<kQ6_K>(x_is_bf16, x, M, K, W, N, bias, act, y, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "qdense: ggml type %d is not implemented", type);
    }
}

}  // namespace gq
