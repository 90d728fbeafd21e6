// Decode GEMV, activation-stationary integer-dot variant (Q4_0, Q8_0, Q4_K; K % 64 == 0,
// K <= 16384).  This is the kernel the bandwidth numbers are quoted on.
//
// Why not plain fp32 FMAs: turning a 4-bit code into an fp32 operand costs more than two
// VALU instructions per weight (mask, convert, fma), and at ~36 T lane-ops/s that alone takes
// as long as streaming the weights from HBM.  Instead the activations are converted ONCE per
// workgroup into fixed-point digit planes that match the packed weight layout, and the
// codes are consumed as they sit in memory by the packed integer dot instructions:
//
//   Q4_0: weights: dword ^ 0x88888888 turns each nibble n into the signed 4-bit value n-8;
//         activations: 20-bit fixed point per 32-block, split into five signed base-16
//         digits; one v_dot8_i32_i4 per digit plane multiplies eight weights.
//   Q8_0: weight bytes are already int8; activations: 22-bit fixed point per 32-block, three
//         signed base-256 limbs; one v_dot4_i32_i8 per limb multiplies four weights.
//   Q4_K: nibbles are split into bytes (two masks per dword) and use the same three limbs;
//         the sub-block minimum multiplies the per-sub-block sum of the activations.
//
// Integer accumulation inside a 32-block is exact; per block the partial sum is converted to
// fp32 once and scaled by d * (activation block scale).  The activation rounding is at most
// 2^-21 (Q4_0) or 2^-23 (Q8_0 / Q4_K) of the block's largest magnitude per element, i.e. the
// same order as fp32 accumulation error over K terms.
//
// Work decomposition: a "unit" is 64 consecutive values of K (two 32-blocks, or one
// 64-value group of a Q4_K super-block).  A wavefront owns a slice of 64 units (4096 values)
// whose digit planes it keeps in registers for its whole life, and streams over many rows
// with a software prefetch PF rows deep, so no LDS traffic and no barrier sit in the steady
// state.  If K needs S > 1 slices, S wavefronts of the workgroup cooperate on each row and
// their partial sums meet in LDS once, at the very end.
#include "blocks.hpp"
#include "common.hpp"

#include <cstdlib>

namespace gq {

namespace {

__device__ __forceinline__ float dpp_quad_max(float v) {
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true)));
    return v;
}
__device__ __forceinline__ float dpp_oct_max(float v) {
    v = dpp_quad_max(v);
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true)));  // row_half_mirror
    return v;
}
__device__ __forceinline__ int dpp_oct_sum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);
    return v;
}

// x is 16-byte aligned on this path (the dispatcher sends other pointers to the generic kernel)
__device__ __forceinline__ float4 ld_x4(const float *x, int i4, bool) { return reinterpret_cast<const float4 *>(x)[i4]; }

// Scale of a 32-block of activations for a fixed-point range of +-qmax.  Blocks that are
// all (nearly) zero quantise to zero; a non-finite block poisons its scale so that the
// affected outputs come out as NaN rather than as a finite wrong number.
__device__ __forceinline__ void block_scale(float amax, float qmax, float &inv, float &scale) {
    if (!(amax >= 0x1p-100f)) {  // zero or tiny
        inv = 0.f;
        scale = 0.f;
    } else if (amax > 3.0e38f) {
        inv = 0.f;
        scale = __builtin_nanf("");
    } else {
        inv = qmax / amax;
        scale = amax / qmax;
    }
}

// ---- activation digit planes in LDS -------------------------------------------------------
// Dword j of unit u lives in LDS word ((j / 4) * nunits + u) * 4 + (j % 4): every lane later
// fetches the planes of its own unit with 16-byte reads, consecutive lanes touching
// consecutive 16-byte slots.
__device__ __forceinline__ int plane_addr(int j, int nunits, int u) { return (((j >> 2) * nunits + u) << 2) + (j & 3); }

// Q4_0: per unit 2 blocks x 4 weight-dwords x 5 digit planes = 40 dwords, then 2 scales
// (44 with padding).  One staging item = the 8 activations that face one weight dword.
constexpr int kNibDwords = 44;
constexpr float kNibQmax = 489000.0f;                 // < 0.4667 * 2^20: fits five balanced hex digits
constexpr float kNibMagic = 12582912.0f + 559240.0f;  // 1.5 * 2^23 + 0x88888

struct NibItem { float4 lo, hi; };

__device__ __forceinline__ NibItem nib_item_load(const float *__restrict__ x, int i, bool aligned) {
    const int b = i >> 2, w = i & 3;
    NibItem it;
    it.lo = ld_x4(x, 8 * b + w, aligned);      // values 4w..4w+3 of the block (low nibbles)
    it.hi = ld_x4(x, 8 * b + 4 + w, aligned);  // values 16+4w.. (high nibbles)
    return it;
}

__device__ __forceinline__ void nib_item_store(const NibItem &it, int i, uint32_t *xs, int nunits) {
    const int b = i >> 2, w = i & 3;
    const float e[8] = {it.lo.x, it.hi.x, it.lo.y, it.hi.y, it.lo.z, it.hi.z, it.lo.w, it.hi.w};  // nibble order
    float amax = 0.f;
    bool nan = false;
#pragma unroll
    for (int p = 0; p < 8; p++) { amax = fmaxf(amax, fabsf(e[p])); nan |= e[p] != e[p]; }
    if (nan) amax = __builtin_inff();  // poison (fmaxf would drop a NaN in the cross-lane maximum)
    amax = dpp_quad_max(amax);         // the four items of a block sit in one quad
    float inv, scale;
    block_scale(amax, kNibQmax, inv, scale);
    uint32_t z[8];
#pragma unroll
    for (int p = 0; p < 8; p++) z[p] = (__builtin_bit_cast(uint32_t, fmaf(e[p], inv, kNibMagic)) & 0xFFFFFu) ^ 0x88888u;
    const int u = b >> 1, h = b & 1;
#pragma unroll
    for (int l = 0; l < 5; l++) {
        uint32_t plane = 0;
#pragma unroll
        for (int p = 0; p < 8; p++) plane |= ((z[p] >> (4 * l)) & 15u) << (4 * p);
        xs[plane_addr((h * 4 + w) * 5 + l, nunits, u)] = plane;
    }
    if (w == 0) xs[plane_addr(40 + h, nunits, u)] = __builtin_bit_cast(uint32_t, scale);
}

// Q8_0 / Q4_K: per unit 2 blocks x 8 runs of four values x 3 limbs = 48 dwords, then
// 2 scales, then 2 block sums (scale * sum of the fixed-point values).  One staging item =
// four consecutive activations.
constexpr int kLimbDwords = 52;
constexpr float kLimbQmax = 4161304.0f;               // 2^22 - 33000
constexpr float kLimbMagic = 12582912.0f + 32896.0f;  // 1.5 * 2^23 + 0x8080

struct LimbItem { float4 v; };

__device__ __forceinline__ LimbItem limb_item_load(const float *__restrict__ x, int i, bool aligned) {
    LimbItem it;
    it.v = ld_x4(x, i, aligned);
    return it;
}

__device__ __forceinline__ void limb_item_store(const LimbItem &it, int i, uint32_t *xs, int nunits) {
    const int b = i >> 3, w = i & 7;
    const float e[4] = {it.v.x, it.v.y, it.v.z, it.v.w};
    float amax = fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3])));
    if (e[0] != e[0] || e[1] != e[1] || e[2] != e[2] || e[3] != e[3]) amax = __builtin_inff();  // poison
    amax = dpp_oct_max(amax);  // the eight items of a block sit in eight consecutive lanes
    float inv, scale;
    block_scale(amax, kLimbQmax, inv, scale);
    uint32_t E[4];
    int xsum = 0;
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const int zs = (int)(__builtin_bit_cast(uint32_t, fmaf(e[p], inv, kLimbMagic)) - 0x4B400000u);  // X + 0x8080
        xsum += zs - 0x8080;
        E[p] = (uint32_t)zs ^ 0x8080u;  // bytes: t0, t1 (signed), t2 (signed), sign fill
    }
    xsum = dpp_oct_sum(xsum);
    const int u = b >> 1, h = b & 1;
#pragma unroll
    for (int l = 0; l < 3; l++) {
        const uint32_t sel = (uint32_t)l | ((uint32_t)(4 + l) << 8);
        const uint32_t p01 = __builtin_amdgcn_perm(E[1], E[0], sel);
        const uint32_t p23 = __builtin_amdgcn_perm(E[3], E[2], sel);
        xs[plane_addr((h * 8 + w) * 3 + l, nunits, u)] = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
    }
    if (w == 0) {
        xs[plane_addr(48 + h, nunits, u)] = __builtin_bit_cast(uint32_t, scale);
        xs[plane_addr(50 + h, nunits, u)] = __builtin_bit_cast(uint32_t, scale * (float)xsum);
    }
}

// ---- per-format lane state: the register-resident activation planes and one row's codes ------

template <int T> struct XS;

template <> struct XS<kQ4_0> {
    static constexpr int kX = kNibDwords;
    struct __attribute__((packed, aligned(4))) Raw { uint32_t v[9]; };
    typedef NibItem Item;
    static constexpr int kItemShift = 3;  // activations per staging item = 8
    static constexpr int kMaxRounds = 4;  // staging items per thread: covers K <= 32 * threads
    static __device__ __forceinline__ Item item_load(const float *x, int i, bool aligned) { return nib_item_load(x, i, aligned); }
    static __device__ __forceinline__ void item_store(const Item &it, int i, uint32_t *xs, int nunits) { nib_item_store(it, i, xs, nunits); }
    static __device__ __forceinline__ void load(Raw &r, const uint8_t *row, int u) {
        r = *reinterpret_cast<const Raw *>(row + (int64_t)u * 36);
    }
    static __device__ __forceinline__ float touch(const Raw &r) { uint32_t a = 0; for (int i = 0; i < 9; i++) a ^= r.v[i]; return (float)a; }
    static __device__ __forceinline__ float dot(const Raw &r, const uint32_t *xq) {
        const uint32_t *v = r.v;
        float out = 0.f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int s[5] = {0, 0, 0, 0, 0};
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t q = (h == 0 ? __builtin_amdgcn_alignbit(v[w + 1], v[w], 16) : v[5 + w]) ^ 0x88888888u;
#pragma unroll
                for (int l = 0; l < 5; l++) s[l] = __builtin_amdgcn_sdot8((int)q, (int)xq[(h * 4 + w) * 5 + l], s[l], false);
            }
            uint32_t t = (uint32_t)s[4];
#pragma unroll
            for (int l = 3; l >= 0; l--) t = (t << 4) + (uint32_t)s[l];  // v_lshl_add_u32
            const float d = half_bits_to_float(h == 0 ? (v[0] & 0xFFFFu) : (v[4] >> 16));
            out = fmaf((float)(int)t, d * __builtin_bit_cast(float, xq[40 + h]), out);
        }
        return out;
    }
};

__device__ __forceinline__ float limb_combine(const int *s) {
    return fmaf((float)s[2], 65536.0f, fmaf((float)s[1], 256.0f, (float)s[0]));
}

template <> struct XS<kQ8_0> {
    static constexpr int kX = kLimbDwords;
    struct __attribute__((packed, aligned(4))) Raw { uint32_t v[17]; };
    typedef LimbItem Item;
    static constexpr int kItemShift = 2;  // activations per staging item = 4
    static constexpr int kMaxRounds = 8;  // staging items per thread: covers K <= 32 * threads
    static __device__ __forceinline__ Item item_load(const float *x, int i, bool aligned) { return limb_item_load(x, i, aligned); }
    static __device__ __forceinline__ void item_store(const Item &it, int i, uint32_t *xs, int nunits) { limb_item_store(it, i, xs, nunits); }
    static __device__ __forceinline__ void load(Raw &r, const uint8_t *row, int u) {
        r = *reinterpret_cast<const Raw *>(row + (int64_t)u * 68);
    }
    static __device__ __forceinline__ float touch(const Raw &r) { uint32_t a = 0; for (int i = 0; i < 17; i++) a ^= r.v[i]; return (float)a; }
    static __device__ __forceinline__ float dot(const Raw &r, const uint32_t *xq) {
        const uint32_t *v = r.v;
        float out = 0.f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int s[3] = {0, 0, 0};
#pragma unroll
            for (int w = 0; w < 8; w++) {
                const uint32_t q = h == 0 ? __builtin_amdgcn_alignbit(v[w + 1], v[w], 16) : v[9 + w];
#pragma unroll
                for (int l = 0; l < 3; l++) s[l] = __builtin_amdgcn_sdot4((int)q, (int)xq[(h * 8 + w) * 3 + l], s[l], false);
            }
            const float d = half_bits_to_float(h == 0 ? (v[0] & 0xFFFFu) : (v[8] >> 16));
            out = fmaf(limb_combine(s), d * __builtin_bit_cast(float, xq[48 + h]), out);
        }
        return out;
    }
};

template <> struct XS<kQ4_K> {
    static constexpr int kX = kLimbDwords;
    struct Raw { uint4 hd, q0, q1; };
    typedef LimbItem Item;
    static constexpr int kItemShift = 2;  // activations per staging item = 4
    static constexpr int kMaxRounds = 8;  // staging items per thread: covers K <= 32 * threads
    static __device__ __forceinline__ Item item_load(const float *x, int i, bool aligned) { return limb_item_load(x, i, aligned); }
    static __device__ __forceinline__ void item_store(const Item &it, int i, uint32_t *xs, int nunits) { limb_item_store(it, i, xs, nunits); }
    // unit u = 4 * super-block + group g: 16-byte header of the super-block + the group's 32 code bytes
    static __device__ __forceinline__ void load(Raw &r, const uint8_t *row, int u) {
        const uint8_t *sb = row + (int64_t)(u >> 2) * 144;
        r.hd = *reinterpret_cast<const uint4 *>(sb);
        const uint4 *q = reinterpret_cast<const uint4 *>(sb + 16 + 32 * (u & 3));
        r.q0 = q[0];
        r.q1 = q[1];
    }
    static __device__ __forceinline__ float touch(const Raw &r) { return (float)(r.hd.x ^ r.hd.y ^ r.hd.z ^ r.hd.w ^ r.q0.x ^ r.q0.y ^ r.q0.z ^ r.q0.w ^ r.q1.x ^ r.q1.y ^ r.q1.z ^ r.q1.w); }
    static __device__ __forceinline__ float dot(const Raw &r, const uint32_t *xq, int g) {
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        const float d = half_bits_to_float(r.hd.x & 0xFFFFu), dmin = half_bits_to_float(r.hd.x >> 16);
        float out = 0.f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int s[3] = {0, 0, 0};
#pragma unroll
            for (int w = 0; w < 8; w++) {
                const uint32_t c = (h == 0 ? q[w] : (q[w] >> 4)) & 0x0F0F0F0Fu;  // four codes as bytes 0..15
#pragma unroll
                for (int l = 0; l < 3; l++) s[l] = __builtin_amdgcn_sdot4((int)c, (int)xq[(h * 8 + w) * 3 + l], s[l], false);
            }
            uint32_t sc, mn;
            q4k_scale_min(r.hd.y, r.hd.z, r.hd.w, 2 * g + h, sc, mn);
            out = fmaf(limb_combine(s), (d * (float)sc) * __builtin_bit_cast(float, xq[48 + h]), out);
            out = fmaf(-(dmin * (float)mn), __builtin_bit_cast(float, xq[50 + h]), out);
        }
        return out;
    }
};

template <int T>
__device__ __forceinline__ float unit_dot(const typename XS<T>::Raw &r, const uint32_t *xq, int u) {
    if constexpr (T == kQ4_K) return XS<T>::dot(r, xq, u & 3);
    else return XS<T>::dot(r, xq);
}

// Sums PF per-lane partials over the 64 lanes at once.  Each halving step both adds and
// routes, so after log2(PF) steps every lane holds one row's partial and the remaining steps
// run on a single register.  Returns in lane l the total of row rowsel(l) where the row a lane
// ends up with is given by its low lane bits: PF=4: row = 2*(l&1) + ((l>>1)&1); PF=2: row = l&1.
template <int PF> struct JointSum;

__device__ __forceinline__ float dpp_xor1(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true)); }
__device__ __forceinline__ float dpp_xor2(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true)); }
__device__ __forceinline__ float dpp_ror4(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, true)); }
__device__ __forceinline__ float dpp_ror8(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, true)); }

// after the quad steps: sum lanes with equal (l & 3) across the wavefront
__device__ __forceinline__ float sum_over_quads(float v) {
    v += dpp_ror4(v);
    v += dpp_ror8(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

template <> struct JointSum<4> {
    static __device__ __forceinline__ float run(const float *p, int lane) {
        const bool b0 = lane & 1, b1 = lane & 2;
        const float a = (b0 ? p[2] : p[0]) + dpp_xor1(b0 ? p[0] : p[2]);
        const float b = (b0 ? p[3] : p[1]) + dpp_xor1(b0 ? p[1] : p[3]);
        const float c = (b1 ? b : a) + dpp_xor2(b1 ? a : b);
        return sum_over_quads(c);
    }
    static __device__ __forceinline__ int row_of_lane(int lane) { return 2 * (lane & 1) + ((lane >> 1) & 1); }
};
template <> struct JointSum<2> {
    static __device__ __forceinline__ float run(const float *p, int lane) {
        const bool b0 = lane & 1;
        float a = (b0 ? p[1] : p[0]) + dpp_xor1(b0 ? p[0] : p[1]);
        a += dpp_xor2(a);
        return sum_over_quads(a);
    }
    static __device__ __forceinline__ int row_of_lane(int lane) { return lane & 1; }
};

// ---- the kernel ---------------------------------------------------------------------------
//
// grid.x workgroups of WAVES wavefronts; wavefront w works on slice (w % S) of the iters
// consecutive rows starting at (blockIdx.x * G + w / S) * iters, with G = WAVES / S.  Rows of a
// wavefront are adjacent in memory on purpose: what the chip has in flight at any moment is
// then one contiguous window of W, whereas rows a large power of two apart land on the same
// HBM channel and bank.
// iters <= 64: lane i of each wavefront ends up with the partial result of its i-th row.
//
// Order of issue matters: vector-memory loads return in order, so the (small, cache-resident)
// activation loads go out first and the PF rows of codes right behind them; the wait for the
// activations then leaves the code loads in flight while the digit planes are being built.

template <int T, int PF>
__device__ __forceinline__ void gemv_xs_body(const float *__restrict__ x, const uint8_t *__restrict__ W,
                                             const float *__restrict__ bias, float *__restrict__ y, int K, int N,
                                             int64_t row_bytes, int S, int iters, int act, int wg, uint32_t *lds) {
    typedef typename XS<T>::Raw Raw;
    typedef typename XS<T>::Item Item;
    constexpr int NX = XS<T>::kX;
    static_assert(NX % 4 == 0, "planes are fetched as 16-byte LDS reads");
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = blockDim.x;
    const int G = (nthreads >> 6) / S;
    const int slice = wave % S, g = wave / S;
    const int nunits = K >> 6;
    const int u = slice * 64 + lane;
    const bool have_unit = u < nunits;
    const int first = (wg * G + g) * iters;  // this wavefront's rows: first .. first + iters - 1
    constexpr bool aligned = true;
    const int nitems = K >> XS<T>::kItemShift;

    // 1. activations of this thread's first staging item, then the first PF rows of codes.
    // Every load below is unconditional (indices are clamped instead of predicated): with
    // straight-line code the compiler can wait for exactly the oldest outstanding load
    // (s_waitcnt vmcnt(n)); a load inside a branch makes it fall back to vmcnt(0), which would
    // serialise the whole prefetch.
    const int last_row = N - 1;
    const int uc = min(u, nunits - 1);
    // Staging items of this thread: tid, tid + nthreads, ... (at most kMaxRounds of them; the
    // host only selects this kernel when that covers K).  The loads sit in blocks of their own
    // so that they are issued here, ahead of the code loads, and not next to their use.
    const int nrounds = (nitems + nthreads - 1) / nthreads;
    constexpr int kMaxRounds = XS<T>::kMaxRounds;
    Item its[kMaxRounds];
#pragma unroll
    for (int m = 0; m < kMaxRounds; m++) {
        if (m < nrounds) its[m] = XS<T>::item_load(x, min(tid + m * nthreads, nitems - 1), aligned);
    }
    // Only the first row goes out before the activations are staged: the texture path takes
    // ~18 cycles per code-load instruction (18 cache lines each), and a wavefront cannot start
    // waiting for its activations before it has queued everything it issues here.
    Raw buf[PF];
    const int my_last = min(first + iters - 1, last_row);
    XS<T>::load(buf[0], W + (int64_t)min(first, my_last) * row_bytes, uc);

    // 2. activations -> digit planes (LDS) -> registers of the owning lanes
#pragma unroll
    for (int m = 0; m < kMaxRounds; m++) {
        if (m < nrounds) {
            const int i = tid + m * nthreads;
            if (i < nitems) XS<T>::item_store(its[m], i, lds, nunits);
        }
    }
#pragma unroll
    for (int j = 1; j < PF; j++) XS<T>::load(buf[j], W + (int64_t)min(first + j, my_last) * row_bytes, uc);
    __syncthreads();
    uint32_t xq[NX];
    {
        const uint4 *l4 = reinterpret_cast<const uint4 *>(lds);
#pragma unroll
        for (int j = 0; j < NX / 4; j++) {
            const uint4 t = l4[j * nunits + uc];
            xq[4 * j] = t.x; xq[4 * j + 1] = t.y; xq[4 * j + 2] = t.z; xq[4 * j + 3] = t.w;
        }
    }

    // 3. stream over the rows, PF at a time.  All groups but the last also fetch the next
    // group's rows (rows past the wavefront's range are clamped to its own last row).
    float mine = 0.f;  // lane i: result of this wavefront's i-th row (its slice of K)
    auto finish_group = [&](const float *part, int i0) {
        constexpr int C = PF >= 4 ? 4 : 2;  // rows reduced together
#pragma unroll
        for (int c = 0; c < PF; c += C) {
            const float tot = JointSum<C>::run(part + c, lane);
            // lane l now holds the total of row i0 + c + row_of_lane(l); hand it to lane i0 + c + r
            const int r = lane - (i0 + c);
            const int src = C == 4 ? (((r & 1) << 1) | ((r >> 1) & 1)) : (r & 1);
            const float got = __shfl(tot, src, 64);
            if (r >= 0 && r < C) mine = got;
        }
    };
    int i0 = 0;
    for (; i0 + PF < iters; i0 += PF) {
        float part[PF];
#pragma unroll
        for (int j = 0; j < PF; j++) {
            const float d = unit_dot<T>(buf[j], xq, u);
            part[j] = (have_unit && first + i0 + j < N) ? d : 0.f;
            XS<T>::load(buf[j], W + (int64_t)min(first + i0 + j + PF, my_last) * row_bytes, uc);
        }
        finish_group(part, i0);
    }
    {
        float part[PF];
#pragma unroll
        for (int j = 0; j < PF; j++) {
            part[j] = 0.f;
            if (i0 + j < iters) {  // uniform: skips the arithmetic of rows this wavefront does not have
                const float d = unit_dot<T>(buf[j], xq, u);
                part[j] = (have_unit && first + i0 + j < N) ? d : 0.f;
            }
        }
        finish_group(part, i0);
    }

    // 4. combine the S slices of every row and write
    if (S == 1) {
        const int row = first + lane;
        if (lane < iters && row < N) y[row] = apply_act(act, mine + (bias ? bias[row] : 0.f));
        return;
    }
    __syncthreads();  // everyone is done reading the planes; reuse LDS for the partial sums
    float *part = reinterpret_cast<float *>(lds);
    if (lane < iters) part[(g * S + slice) * 64 + lane] = mine;
    __syncthreads();
    if (slice == 0 && lane < iters) {
        const int row = first + lane;
        if (row < N) {
            float t = 0.f;
            for (int s = 0; s < S; s++) t += part[(g * S + s) * 64 + lane];
            y[row] = apply_act(act, t + (bias ? bias[row] : 0.f));
        }
    }
}

template <int T, int PF, int MAXT>
__global__ __launch_bounds__(MAXT) void gemv_xs_kernel(const float *__restrict__ X, const uint8_t *__restrict__ W,
                                                       const float *__restrict__ bias, float *__restrict__ Y, int K,
                                                       int N, int64_t row_bytes, int S, int iters, int act) {
    extern __shared__ uint32_t lds[];
    gemv_xs_body<T, PF>(X + (int64_t)blockIdx.y * K, W, bias, Y + (int64_t)blockIdx.y * N, K, N, row_bytes, S, iters, act,
                        (int)blockIdx.x, lds);
}

// Several independent batch-1 problems of one format in a single launch: workgroups
// [wg_begin, next wg_begin) belong to problem i.  This is how the projections of a decoder
// layer that do not depend on each other (q/k/v, gate/up) share one submission.
constexpr int kMaxBatch = 8;
struct XsProblem {
    const float *x;
    const uint8_t *W;
    const float *bias;
    float *y;
    int64_t row_bytes;
    int K, N, S, iters, act, wg_begin;
};
struct XsBatch {
    int count;
    XsProblem p[kMaxBatch];
};

template <int T, int PF, int MAXT>
__global__ __launch_bounds__(MAXT) void gemv_xs_batch_kernel(const XsBatch b) {
    extern __shared__ uint32_t lds[];
    int i = 0;
#pragma unroll
    for (int j = 1; j < kMaxBatch; j++)
        if (j < b.count && (int)blockIdx.x >= b.p[j].wg_begin) i = j;
    const XsProblem &q = b.p[i];
    gemv_xs_body<T, PF>(q.x, q.W, q.bias, q.y, q.K, q.N, q.row_bytes, q.S, q.iters, q.act, (int)blockIdx.x - q.wg_begin, lds);
}

struct Plan { int waves, S, G, wgs, iters; };

// Picks workgroup size, slices and grid.  GOMLX_HIPQ_GEMV_XS="wgs_per_cu,waves" overrides the
// built-in choice (tuning runs only).
Plan make_plan(int64_t K, int64_t N, int max_waves) {
    static const int env_wgs = [] { const char *e = std::getenv("GOMLX_HIPQ_GEMV_XS"); int a = 0, b = 0; return (e && std::sscanf(e, "%d,%d", &a, &b) == 2) ? a : 0; }();
    static const int env_waves = [] { const char *e = std::getenv("GOMLX_HIPQ_GEMV_XS"); int a = 0, b = 0; return (e && std::sscanf(e, "%d,%d", &a, &b) == 2) ? b : 0; }();
    Plan p;
    const int nunits = (int)(K >> 6);
    int S = 1;
    while (S * 64 < nunits) S <<= 1;
    p.S = S;
    p.waves = env_waves ? env_waves : 8;
    if (p.waves > max_waves) p.waves = max_waves;
    if (p.waves < S) p.waves = S;
    while ((int64_t)p.waves * 64 * 32 < K) p.waves <<= 1;  // staging: at most K / 32 threads' worth of items
    p.G = p.waves / S;
    const int cus = device_cu_count();
    const int64_t target_wgs = (int64_t)cus * (env_wgs ? env_wgs : 1);  // one workgroup per CU measured best
    int64_t slots = target_wgs * p.G;
    int64_t iters = (N + slots - 1) / slots;
    if (iters < 1) iters = 1;
    if (iters > 64) iters = 64;
    p.iters = (int)iters;
    p.wgs = (int)((N + iters * p.G - 1) / (iters * p.G));
    return p;
}

template <int T, int PF, int MAXT>
int launch_xs(const Plan &p, const float *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act,
              float *y, hipStream_t s) {
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    const int nunits = (int)(K >> 6);
    size_t shmem = (size_t)(T == kQ4_0 ? kNibDwords : kLimbDwords) * nunits * sizeof(uint32_t);
    const size_t part_bytes = (size_t)p.waves * 64 * sizeof(float);
    if (shmem < part_bytes) shmem = part_bytes;
    return launch(gemv_xs_kernel<T, PF, MAXT>, dim3((unsigned)p.wgs, (unsigned)M), dim3(p.waves * 64), shmem, s, x, W, bias, y,
                  (int)K, (int)N, row_bytes, p.S, p.iters, act);
}

// Prefetch depth = rows a wavefront keeps in flight: as many as it has, up to PFMAX (register
// budget of the format).  Waves are limited to 8 per workgroup (512 threads) so that the deep
// variants may use up to 256 VGPRs.
template <int T, int PFMAX>
int launch_depth(const float *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
                 hipStream_t s) {
    const Plan p = make_plan(K, N, 8);
    if (p.iters <= 2 || PFMAX == 2) return launch_xs<T, 2, 512>(p, x, M, K, W, N, bias, act, y, s);
    if (p.iters <= 4 || PFMAX == 4) return launch_xs<T, 4, 512>(p, x, M, K, W, N, bias, act, y, s);
    return launch_xs<T, PFMAX, 512>(p, x, M, K, W, N, bias, act, y, s);
}

template <int T>
size_t xs_lds_bytes(int64_t K, int waves) {
    size_t shmem = (size_t)(T == kQ4_0 ? kNibDwords : kLimbDwords) * (size_t)(K >> 6) * sizeof(uint32_t);
    const size_t part_bytes = (size_t)waves * 64 * sizeof(float);
    return shmem < part_bytes ? part_bytes : shmem;
}

// One launch for `count` batch-1 problems: the chip's workgroup slots are shared out in proportion
// to each problem's weight bytes, so every CU streams for about the same time.
template <int T>
int launch_xs_batch(int count, const XsProblem *in, hipStream_t s) {
    XsBatch b;
    b.count = count;
    const int cus = device_cu_count();
    double total = 0.0;
    for (int i = 0; i < count; i++) total += (double)in[i].row_bytes * in[i].N;
    size_t shmem = 0;
    int wg = 0;
    for (int i = 0; i < count; i++) {
        XsProblem q = in[i];
        int S = 1;
        while (S * 64 < (q.K >> 6)) S <<= 1;
        const int waves = 8, G = waves / S;
        int64_t share = (int64_t)((double)cus * ((double)q.row_bytes * q.N) / total + 0.5);
        if (share < 1) share = 1;
        int64_t iters = (q.N + share * G - 1) / (share * G);
        if (iters < 1) iters = 1;
        if (iters > 64) iters = 64;
        q.S = S;
        q.iters = (int)iters;
        q.wg_begin = wg;
        wg += (int)((q.N + iters * G - 1) / (iters * G));
        b.p[i] = q;
        const size_t need = xs_lds_bytes<T>(q.K, waves);
        if (need > shmem) shmem = need;
    }
    return launch(gemv_xs_batch_kernel<T, 4, 512>, dim3((unsigned)wg), dim3(512), shmem, s, b);
}

}  // namespace

int launch_gemv_xs_batch(int type, int count, const XsBatchItem *items, hipStream_t s) {
    if (count < 1 || count > kMaxBatch) return fail(GQ_ERR_INVALID, "gemv batch: %d problems (1..%d supported per launch)", count, kMaxBatch);
    XsProblem p[kMaxBatch];
    for (int i = 0; i < count; i++) {
        const XsBatchItem &it = items[i];
        p[i].x = it.x; p[i].W = it.W; p[i].bias = it.bias; p[i].y = it.y;
        p[i].K = (int)it.K; p[i].N = (int)it.N; p[i].act = it.act;
        p[i].row_bytes = (int64_t)gq_row_bytes(type, it.K);
        p[i].S = p[i].iters = p[i].wg_begin = 0;
    }
    switch (type) {
    case kQ4_0: return launch_xs_batch<kQ4_0>(count, p, s);
    case kQ8_0: return launch_xs_batch<kQ8_0>(count, p, s);
    case kQ4_K: return launch_xs_batch<kQ4_K>(count, p, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv batch: ggml type %d is not implemented", type);
    }
}

bool gemv_xs_supported(int type, int64_t K, int64_t N, const void *x) {
    if (reinterpret_cast<uintptr_t>(x) & 15) return false;
    if (type != kQ4_0 && type != kQ8_0 && type != kQ4_K) return false;
    return K % 64 == 0 && K <= 16384 && N <= (int64_t)INT32_MAX / 2;
}

int launch_gemv_xs(int type, const float *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias,
                   int act, float *y, hipStream_t s) {
    switch (type) {
    case kQ4_0: return launch_depth<kQ4_0, 4>(x, M, K, W, N, bias, act, y, s);
    case kQ8_0: return launch_depth<kQ8_0, 4>(x, M, K, W, N, bias, act, y, s);
    case kQ4_K: return launch_depth<kQ4_K, 4>(x, M, K, W, N, bias, act, y, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv_xs: ggml type %d is not implemented", type);
    }
}

}  // namespace gq
