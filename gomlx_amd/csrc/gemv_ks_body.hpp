// Decode GEMV, K-sliced integer-dot kernels with wavefront-local activation staging
// (Q4_0, Q8_0, Q4_K, Q6_K, IQ4_NL; K % 256 == 0).
//
// The activation-stationary kernel of gemv_xs.hip lets every wavefront see all of K, so its
// workgroup has to convert the whole activation vector together and meet at a barrier before the
// first code byte can be used; on a 5-10 us kernel that prologue is a quarter of the run time.
// Here a wavefront owns one 512-value slice of K (16 blocks of 32) instead: its 64 lanes convert
// 8 activations each, exchange the fixed-point planes through a private piece of LDS (no
// barrier: LDS operations of one wavefront execute in order) and start on the codes as soon as
// their own 2 KB of x have arrived.  The wavefronts of a workgroup cover the slices of the same
// rows (slice w, w + waves, ...: one more for the first few when the count does not divide; a last
// half slice when K is an odd multiple of 256 runs with zero activations for its missing half) and
// add their partial sums in LDS once, at the very end.
//
// Lane l = 8 * rg + c works on row (8 * it + rg) of the workgroup and on 64 values of the slice:
//   Q4_0: blocks 2c, 2c+1: 36 bytes at a 4-byte-aligned address;
//   Q8_0: blocks 2c, 2c+1: 68 bytes at a 4-byte-aligned address;
//   Q4_K: super-block c / 4 of the slice, 64-value group c % 4: the 16-byte header and 32 code bytes;
//   Q6_K: super-block c / 4, half (c / 2) % 2, and of each of the half's four 32-value quadrants
//         the 16 values (c % 2) * 16 ..: 16 + 16 bytes of low nibbles, 16 bytes of high bit pairs,
//         the half's 8 scales and d.
// A load instruction therefore covers 8 rows x one contiguous slice (288, 544 or 420 bytes).
//
// Activation fixed point: 16 bits per 32 values.  Q4_0 uses four balanced base-16 digits (digit
// planes in the nibble order of a weight dword, one v_dot8_i32_i4 per plane); Q8_0 and Q4_K use
// two signed base-256 limbs (one v_dot4_i32_i8 per limb).  The rounding is at most 2^-16 of the
// 32 values' largest magnitude per element; over K = 4096 random terms that is a relative output
// error of a few 1e-5, well inside the 1e-3 bound of this path.
#pragma once

#include "blocks.hpp"
#include "common.hpp"

#include <cstdlib>

namespace gq {

namespace {

constexpr float kQmax4 = 30500.0f;                   // |q| <= 30583 fits four balanced hex digits
constexpr float kMagic4 = 12582912.0f + 34952.0f;    // 1.5 * 2^23 + 0x8888
constexpr float kQmaxL = 32500.0f;                   // |q| <= 32639 fits two balanced base-256 limbs
constexpr float kMagicL = 12582912.0f + 32896.0f;    // 1.5 * 2^23 + 0x8080
constexpr int kSliceValues = 512;
constexpr int kMaxItersKs = 64;                      // rows per workgroup <= 512

__device__ __forceinline__ float ks_quad_max(float v) {
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true)));
    return v;
}
// sum over the 8 lanes of an aligned group of 8 (every lane ends up with the total)
__device__ __forceinline__ float ks_oct_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    return v;
}

// sum over the 4 lanes of a quad (integer)
__device__ __forceinline__ int ks_quad_sum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);
    return v;
}

struct XPair { float4 lo, hi; };

// bf16 -> fp32 is a shift; two values per dword
__device__ __forceinline__ float bf16_lo(uint32_t u) { return __builtin_bit_cast(float, u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __builtin_bit_cast(float, u & 0xFFFF0000u); }

// Scale of 32 activations for a fixed-point range of +-qmax.  All-zero groups quantise to zero; a
// non-finite group poisons its scale so that the affected outputs come out as NaN.
__device__ __forceinline__ void ks_scale(const float *e, float qmax, float &inv, float &scale) {
    float amax = 0.f;
    bool nan = false;
#pragma unroll
    for (int p = 0; p < 8; p++) { amax = fmaxf(amax, fabsf(e[p])); nan |= e[p] != e[p]; }
    if (nan) amax = __builtin_inff();  // fmaxf would drop a NaN in the cross-lane maximum
    amax = ks_quad_max(amax);          // the four lanes that hold 32 consecutive values form a quad
    if (!(amax >= 0x1p-100f)) { inv = 0.f; scale = 0.f; }
    else if (amax > 3.0e38f) { inv = 0.f; scale = __builtin_nanf(""); }
    else { inv = qmax / amax; scale = amax / qmax; }
}

// What a lane publishes for the 8 activations it converts: four plane dwords, the scale of their
// 32-value group and (limb formats) scale * sum of the group's fixed-point values.
struct Staged { uint4 planes; float scale, sum; };

// ---- per-format traits -----------------------------------------------------------------------------
template <int T> struct KS;

template <> struct KS<kQ4_0> {
    static constexpr int kSliceBytes = 288;
    // where a lane finds what it needs of the staged slice: plane vector i (0..7), scale i, sum i
    static constexpr int kScales = 2, kSumSpan = 0;
    static __device__ __forceinline__ int plane_idx(int c, int i) { return 8 * c + i; }
    static __device__ __forceinline__ int scale_idx(int c, int i) { return 2 * c + i; }
    static __device__ __forceinline__ int sum_idx(int c, int i) { return 2 * c + i; }
    struct __attribute__((packed, aligned(4))) Raw { uint32_t v[9]; };
    static __device__ __forceinline__ int lane_offset(int c) { return c * 36; }
    static __device__ __forceinline__ void load(Raw &r, const uint8_t *p) { r = *reinterpret_cast<const Raw *>(p); }
    // the 8 activations that face weight dword (lane & 3) of block (lane >> 2) of the slice
    static __device__ __forceinline__ void x_fetch(const float *__restrict__ xs, int lane, uint4 &a, uint4 &b) {
        const uint4 *x4 = reinterpret_cast<const uint4 *>(xs) + (lane >> 2) * 8 + (lane & 3);
        a = x4[0];  // values 4w .. 4w+3 of the block (low nibbles of code bytes 4w .. 4w+3)
        b = x4[4];  // values 16+4w .. (high nibbles)
    }
    static __device__ __forceinline__ uint4 x_fetch_bf16(const uint16_t *__restrict__ xs, int lane) {
        const uint2 *x2 = reinterpret_cast<const uint2 *>(xs) + (lane >> 2) * 8 + (lane & 3);
        const uint2 a = x2[0], b = x2[4];
        return make_uint4(a.x, a.y, b.x, b.y);
    }
    static __device__ __forceinline__ XPair x_widen_bf16(const uint4 &u) {
        XPair p;
        p.lo = make_float4(bf16_lo(u.x), bf16_hi(u.x), bf16_lo(u.y), bf16_hi(u.y));
        p.hi = make_float4(bf16_lo(u.z), bf16_hi(u.z), bf16_lo(u.w), bf16_hi(u.w));
        return p;
    }
    // nibble p of plane d = digit d of the activation facing nibble p of the weight dword
    static __device__ __forceinline__ Staged stage(const XPair &xp) {
        const float e[8] = {xp.lo.x, xp.hi.x, xp.lo.y, xp.hi.y, xp.lo.z, xp.hi.z, xp.lo.w, xp.hi.w};  // nibble order
        Staged st;
        float inv;
        ks_scale(e, kQmax4, inv, st.scale);
        st.sum = 0.f;
        uint32_t z[8];
#pragma unroll
        for (int p = 0; p < 8; p++) z[p] = __builtin_bit_cast(uint32_t, fmaf(e[p], inv, kMagic4));  // low 16 bits: q + 0x8888
        // byte 0 of z = digits 0,1; byte 1 = digits 2,3.  Gather the bytes of the even and of the
        // odd nibble positions, then interleave nibbles.
        const uint32_t ga = __builtin_amdgcn_perm(z[2], z[0], 0x05010400u), gb = __builtin_amdgcn_perm(z[6], z[4], 0x05010400u);
        const uint32_t gc = __builtin_amdgcn_perm(z[3], z[1], 0x05010400u), gd = __builtin_amdgcn_perm(z[7], z[5], 0x05010400u);
        const uint32_t e0 = __builtin_amdgcn_perm(gb, ga, 0x05040100u) ^ 0x88888888u, e1 = __builtin_amdgcn_perm(gb, ga, 0x07060302u) ^ 0x88888888u;
        const uint32_t o0 = __builtin_amdgcn_perm(gd, gc, 0x05040100u) ^ 0x88888888u, o1 = __builtin_amdgcn_perm(gd, gc, 0x07060302u) ^ 0x88888888u;
        constexpr uint32_t m = 0x0F0F0F0Fu;
        st.planes.x = (e0 & m) | ((o0 & m) << 4);
        st.planes.y = ((e0 >> 4) & m) | (o0 & ~m);
        st.planes.z = (e1 & m) | ((o1 & m) << 4);
        st.planes.w = ((e1 >> 4) & m) | (o1 & ~m);
        return st;
    }
    // xq[4 h + w] = planes facing dword w of block h
    static __device__ __forceinline__ float dot(const Raw &r, const uint4 *xq, const float *xsc, const float *, int) {
        const uint32_t *v = r.v;
        float out = 0.f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int s0 = 0, s1 = 0, s2 = 0, s3 = 0;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const int q = (int)((h == 0 ? __builtin_amdgcn_alignbit(v[w + 1], v[w], 16) : v[5 + w]) ^ 0x88888888u);
                const uint4 &pl = xq[h * 4 + w];
                s0 = __builtin_amdgcn_sdot8(q, (int)pl.x, s0, false);
                s1 = __builtin_amdgcn_sdot8(q, (int)pl.y, s1, false);
                s2 = __builtin_amdgcn_sdot8(q, (int)pl.z, s2, false);
                s3 = __builtin_amdgcn_sdot8(q, (int)pl.w, s3, false);
            }
            uint32_t t = (uint32_t)s3;
            t = (t << 4) + (uint32_t)s2;  // v_lshl_add_u32
            t = (t << 4) + (uint32_t)s1;
            t = (t << 4) + (uint32_t)s0;
            const float d = half_bits_to_float(h == 0 ? (v[0] & 0xFFFFu) : (v[4] >> 16));
            out = fmaf((float)(int)t, d * xsc[h], out);
        }
        return out;
    }
};

// Q8_0 and Q4_K: lane l converts activations 8l .. 8l+7 of the slice, i.e. the values facing dwords
// 2j, 2j+1 (j = l & 3) of 32-value group l >> 2.  planes = {limb0, limb1 of dword 2j, limb0, limb1 of
// dword 2j+1}, byte i of a plane = limb of value 4 * dword + i.
__device__ __forceinline__ void limb_x_fetch(const float *__restrict__ xs, int lane, uint4 &a, uint4 &b) {
    const uint4 *x4 = reinterpret_cast<const uint4 *>(xs) + 2 * lane;
    a = x4[0];
    b = x4[1];
}
__device__ __forceinline__ uint4 limb_x_fetch_bf16(const uint16_t *__restrict__ xs, int lane) {
    return reinterpret_cast<const uint4 *>(xs)[lane];
}
__device__ __forceinline__ XPair limb_x_widen_bf16(const uint4 &a) {
    XPair p;
    p.lo = make_float4(bf16_lo(a.x), bf16_hi(a.x), bf16_lo(a.y), bf16_hi(a.y));
    p.hi = make_float4(bf16_lo(a.z), bf16_hi(a.z), bf16_lo(a.w), bf16_hi(a.w));
    return p;
}
// SUM16: the published sum covers the 16 values of a lane pair and is pre-multiplied by -32 (the
// offset of a Q6_K code); otherwise it covers the 32 values of the quad.
template <bool SUM16 = false>
__device__ __forceinline__ Staged limb_stage(const XPair &xp) {
    const float e[8] = {xp.lo.x, xp.lo.y, xp.lo.z, xp.lo.w, xp.hi.x, xp.hi.y, xp.hi.z, xp.hi.w};
    Staged st;
    float inv;
    ks_scale(e, kQmaxL, inv, st.scale);
    uint32_t z[8];
    int xsum = 0;
#pragma unroll
    for (int p = 0; p < 8; p++) {
        const int zs = (int)(__builtin_bit_cast(uint32_t, fmaf(e[p], inv, kMagicL)) - 0x4B400000u);  // q + 0x8080
        xsum += zs - 0x8080;
        z[p] = (uint32_t)zs;
    }
    if constexpr (SUM16) {
        xsum += __builtin_amdgcn_update_dpp(0, xsum, 0xB1, 0xF, 0xF, true);
        st.sum = -32.f * st.scale * (float)xsum;
    } else {
        xsum = ks_quad_sum(xsum);
        st.sum = st.scale * (float)xsum;
    }
    const uint32_t a01 = __builtin_amdgcn_perm(z[1], z[0], 0x05010400u), a23 = __builtin_amdgcn_perm(z[3], z[2], 0x05010400u);
    const uint32_t b01 = __builtin_amdgcn_perm(z[5], z[4], 0x05010400u), b23 = __builtin_amdgcn_perm(z[7], z[6], 0x05010400u);
    st.planes.x = __builtin_amdgcn_perm(a23, a01, 0x05040100u) ^ 0x80808080u;
    st.planes.y = __builtin_amdgcn_perm(a23, a01, 0x07060302u) ^ 0x80808080u;
    st.planes.z = __builtin_amdgcn_perm(b23, b01, 0x05040100u) ^ 0x80808080u;
    st.planes.w = __builtin_amdgcn_perm(b23, b01, 0x07060302u) ^ 0x80808080u;
    return st;
}
// planes of dword w (0..7) of group h: limb 0 and limb 1
__device__ __forceinline__ void limb_planes(const uint4 *xq, int h, int w, int &p0, int &p1) {
    const uint4 &pl = xq[h * 4 + (w >> 1)];
    p0 = (int)((w & 1) ? pl.z : pl.x);
    p1 = (int)((w & 1) ? pl.w : pl.y);
}

template <> struct KS<kQ8_0> {
    static constexpr int kSliceBytes = 544;
    // where a lane finds what it needs of the staged slice: plane vector i (0..7), scale i, sum i
    static constexpr int kScales = 2, kSumSpan = 0;
    static __device__ __forceinline__ int plane_idx(int c, int i) { return 8 * c + i; }
    static __device__ __forceinline__ int scale_idx(int c, int i) { return 2 * c + i; }
    static __device__ __forceinline__ int sum_idx(int c, int i) { return 2 * c + i; }
    struct __attribute__((packed, aligned(4))) Raw { uint32_t v[17]; };
    static __device__ __forceinline__ int lane_offset(int c) { return c * 68; }
    static __device__ __forceinline__ void load(Raw &r, const uint8_t *p) { r = *reinterpret_cast<const Raw *>(p); }
    static __device__ __forceinline__ void x_fetch(const float *__restrict__ xs, int lane, uint4 &a, uint4 &b) { limb_x_fetch(xs, lane, a, b); }
    static __device__ __forceinline__ uint4 x_fetch_bf16(const uint16_t *__restrict__ xs, int lane) { return limb_x_fetch_bf16(xs, lane); }
    static __device__ __forceinline__ XPair x_widen_bf16(const uint4 &u) { return limb_x_widen_bf16(u); }
    static __device__ __forceinline__ Staged stage(const XPair &xp) { return limb_stage(xp); }
    static __device__ __forceinline__ float dot(const Raw &r, const uint4 *xq, const float *xsc, const float *, int) {
        const uint32_t *v = r.v;
        float out = 0.f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int s0 = 0, s1 = 0;
#pragma unroll
            for (int w = 0; w < 8; w++) {
                const int q = (int)(h == 0 ? __builtin_amdgcn_alignbit(v[w + 1], v[w], 16) : v[9 + w]);
                int p0, p1;
                limb_planes(xq, h, w, p0, p1);
                s0 = __builtin_amdgcn_sdot4(q, p0, s0, false);
                s1 = __builtin_amdgcn_sdot4(q, p1, s1, false);
            }
            const int t = (s1 << 8) + s0;
            const float d = half_bits_to_float(h == 0 ? (v[0] & 0xFFFFu) : (v[8] >> 16));
            out = fmaf((float)t, d * xsc[h], out);
        }
        return out;
    }
};

// IQ4_NL: the byte layout of Q4_0 (lane c: blocks 2c, 2c+1, 36 bytes), but the nibbles index a
// 16-entry code book of int8 values, looked up four at a time with byte permutes; the dot products
// then run on the two signed byte limbs like Q8_0.  Low nibbles of code dword w face values
// 4w .. 4w+3 of the block (plane dword w), high nibbles values 16+4w .. (plane dword 4+w).
template <> struct KS<kIQ4_NL> {
    static constexpr int kSliceBytes = 288;
    static constexpr int kScales = 2, kSumSpan = 0;
    static __device__ __forceinline__ int plane_idx(int c, int i) { return 8 * c + i; }
    static __device__ __forceinline__ int scale_idx(int c, int i) { return 2 * c + i; }
    static __device__ __forceinline__ int sum_idx(int c, int i) { return 2 * c + i; }
    struct __attribute__((packed, aligned(4))) Raw { uint32_t v[9]; };
    static __device__ __forceinline__ int lane_offset(int c) { return c * 36; }
    static __device__ __forceinline__ void load(Raw &r, const uint8_t *p) { r = *reinterpret_cast<const Raw *>(p); }
    static __device__ __forceinline__ void x_fetch(const float *__restrict__ xs, int lane, uint4 &a, uint4 &b) { limb_x_fetch(xs, lane, a, b); }
    static __device__ __forceinline__ uint4 x_fetch_bf16(const uint16_t *__restrict__ xs, int lane) { return limb_x_fetch_bf16(xs, lane); }
    static __device__ __forceinline__ XPair x_widen_bf16(const uint4 &u) { return limb_x_widen_bf16(u); }
    static __device__ __forceinline__ Staged stage(const XPair &xp) { return limb_stage(xp); }
    // four code-book entries (int8, as bytes) for the four indices 0..15 in the bytes of idx
    static __device__ __forceinline__ int book(uint32_t idx) {
        const uint32_t t0 = 0xBFAD9881u, t1 = 0xF6EADDCFu, t2 = 0x26190D01u, t3 = 0x71594535u;  // -127 .. 113, four per dword
        const uint32_t low3 = idx & 0x07070707u;
        const uint32_t lo = __builtin_amdgcn_perm(t1, t0, low3), hi = __builtin_amdgcn_perm(t3, t2, low3);
        return (int)__builtin_amdgcn_perm(hi, lo, 0x03020100u | ((idx & 0x08080808u) >> 1));  // byte i from hi when bit 3 of index i is set
    }
    static __device__ __forceinline__ float dot(const Raw &r, const uint4 *xq, const float *xsc, const float *, int) {
        const uint32_t *v = r.v;
        float out = 0.f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int s0 = 0, s1 = 0;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t q = h == 0 ? __builtin_amdgcn_alignbit(v[w + 1], v[w], 16) : v[5 + w];
                const int lo = book(q & 0x0F0F0F0Fu), hi = book((q >> 4) & 0x0F0F0F0Fu);
                int p0, p1;
                limb_planes(xq, h, w, p0, p1);
                s0 = __builtin_amdgcn_sdot4(lo, p0, s0, false);
                s1 = __builtin_amdgcn_sdot4(lo, p1, s1, false);
                limb_planes(xq, h, 4 + w, p0, p1);
                s0 = __builtin_amdgcn_sdot4(hi, p0, s0, false);
                s1 = __builtin_amdgcn_sdot4(hi, p1, s1, false);
            }
            const int t = (s1 << 8) + s0;
            const float d = half_bits_to_float(h == 0 ? (v[0] & 0xFFFFu) : (v[4] >> 16));
            out = fmaf((float)t, d * xsc[h], out);
        }
        return out;
    }
};

template <> struct KS<kQ4_K> {
    static constexpr int kSliceBytes = 288;  // two super-blocks
    // where a lane finds what it needs of the staged slice: plane vector i (0..7), scale i, sum i
    static constexpr int kScales = 2, kSumSpan = 32;
    static __device__ __forceinline__ int plane_idx(int c, int i) { return 8 * c + i; }
    static __device__ __forceinline__ int scale_idx(int c, int i) { return 2 * c + i; }
    static __device__ __forceinline__ int sum_idx(int c, int i) { return 2 * c + i; }
    struct Raw { uint4 hd, q0, q1; };
    static __device__ __forceinline__ int lane_offset(int c) { return (c >> 2) * 144; }
    static __device__ __forceinline__ void load(Raw &r, const uint8_t *sb, int c) {
        r.hd = *reinterpret_cast<const uint4 *>(sb);
        const uint4 *q = reinterpret_cast<const uint4 *>(sb + 16 + 32 * (c & 3));
        r.q0 = q[0];
        r.q1 = q[1];
    }
    static __device__ __forceinline__ void x_fetch(const float *__restrict__ xs, int lane, uint4 &a, uint4 &b) { limb_x_fetch(xs, lane, a, b); }
    static __device__ __forceinline__ uint4 x_fetch_bf16(const uint16_t *__restrict__ xs, int lane) { return limb_x_fetch_bf16(xs, lane); }
    static __device__ __forceinline__ XPair x_widen_bf16(const uint4 &u) { return limb_x_widen_bf16(u); }
    static __device__ __forceinline__ Staged stage(const XPair &xp) { return limb_stage(xp); }
    static __device__ __forceinline__ float dot(const Raw &r, const uint4 *xq, const float *xsc, const float *xsm, int c) {
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        const float d = half_bits_to_float(r.hd.x & 0xFFFFu), dmin = half_bits_to_float(r.hd.x >> 16);
        const int g = c & 3;
        float out = 0.f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int s0 = 0, s1 = 0;
#pragma unroll
            for (int w = 0; w < 8; w++) {
                const int cw = (int)((h == 0 ? q[w] : (q[w] >> 4)) & 0x0F0F0F0Fu);  // four codes as bytes 0..15
                int p0, p1;
                limb_planes(xq, h, w, p0, p1);
                s0 = __builtin_amdgcn_sdot4(cw, p0, s0, false);
                s1 = __builtin_amdgcn_sdot4(cw, p1, s1, false);
            }
            const int t = (s1 << 8) + s0;
            uint32_t sc, mn;
            q4k_scale_min(r.hd.y, r.hd.z, r.hd.w, 2 * g + h, sc, mn);
            out = fmaf((float)t, (d * (float)sc) * xsc[h], out);
            out = fmaf(-(dmin * (float)mn), xsm[h], out);
        }
        return out;
    }
};


// Q6_K: w = d * sc[16-value run] * (code - 32), code = low nibble | two high bits << 4.  The
// -32 is applied through the activation sums of the run, so the codes stay unsigned bytes.
template <> struct KS<kQ6_K> {
    static constexpr int kSliceBytes = 420;  // two super-blocks
    static constexpr int kScales = 4, kSumSpan = 16;
    // c = 4 * sb + 2 * half + pp; quadrant qd's run is values 32 * qd + 16 * pp .. of the half
    static __device__ __forceinline__ int plane_idx(int c, int i) { return 8 * (c & ~1) + 2 * (c & 1) + 4 * (i >> 1) + (i & 1); }
    static __device__ __forceinline__ int scale_idx(int c, int i) { return 2 * (c & ~1) + i; }
    static __device__ __forceinline__ int sum_idx(int c, int i) { return 4 * (c & ~1) + 2 * i + (c & 1); }
    struct __attribute__((packed, aligned(2))) U4 { uint32_t v[4]; };
    struct __attribute__((packed, aligned(2))) U2 { uint32_t v[2]; };
    struct Raw { U4 a, b, h; U2 sc; uint32_t d; };
    static __device__ __forceinline__ int lane_offset(int c) { return (c >> 2) * 210; }
    static __device__ __forceinline__ void load(Raw &r, const uint8_t *sb, int c) {
        const int half = (c >> 1) & 1, pp = c & 1;
        const uint8_t *ql = sb + 64 * half + 16 * pp;
        r.a = *reinterpret_cast<const U4 *>(ql);
        r.b = *reinterpret_cast<const U4 *>(ql + 32);
        r.h = *reinterpret_cast<const U4 *>(sb + 128 + 32 * half + 16 * pp);
        r.sc = *reinterpret_cast<const U2 *>(sb + 192 + 8 * half);
        r.d = *reinterpret_cast<const uint16_t *>(sb + 208);
    }
    static __device__ __forceinline__ void x_fetch(const float *__restrict__ xs, int lane, uint4 &a, uint4 &b) { limb_x_fetch(xs, lane, a, b); }
    static __device__ __forceinline__ uint4 x_fetch_bf16(const uint16_t *__restrict__ xs, int lane) { return limb_x_fetch_bf16(xs, lane); }
    static __device__ __forceinline__ XPair x_widen_bf16(const uint4 &u) { return limb_x_widen_bf16(u); }
    static __device__ __forceinline__ Staged stage(const XPair &xp) { return limb_stage<true>(xp); }
    // xq[2 qd + e] = planes of values 8 e .. 8 e + 7 of quadrant qd's run; xsc[qd] the scale of the
    // quadrant's activations, xsm[qd] = -32 * (sum of the run's activations as quantised)
    static __device__ __forceinline__ float dot(const Raw &r, const uint4 *xq, const float *xsc, const float *xsm, int c) {
        const int sc_shift = 8 * (c & 1);
        float out = 0.f;
#pragma unroll
        for (int qd = 0; qd < 4; qd++) {
            int s0 = 0, s1 = 0;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t src = (qd & 1) ? r.b.v[w] : r.a.v[w];
                const uint32_t lo = ((qd >> 1) ? (src >> 4) : src) & 0x0F0F0F0Fu;
                const uint32_t hv = r.h.v[w];
                const uint32_t hs = qd == 0 ? (hv << 4) : qd == 1 ? (hv << 2) : qd == 2 ? hv : (hv >> 2);
                const int code = (int)((hs & 0x30303030u) | lo);
                const uint4 &pl = xq[2 * qd + (w >> 1)];
                s0 = __builtin_amdgcn_sdot4(code, (int)((w & 1) ? pl.z : pl.x), s0, false);
                s1 = __builtin_amdgcn_sdot4(code, (int)((w & 1) ? pl.w : pl.y), s1, false);
            }
            const int t = (s1 << 8) + s0;
            const int sc = __builtin_amdgcn_sbfe((int)r.sc.v[qd >> 1], 16 * (qd & 1) + sc_shift, 8);
            out = fmaf((float)sc, fmaf((float)t, xsc[qd], xsm[qd]), out);
        }
        return out * half_bits_to_float(r.d & 0xFFFFu);
    }
};

// Activation rows a pass can serve at once: the planes of four rows fit the register file next to
// the loads in flight, except for Q6_K (four scale and sum registers per row, the widest decoder).
template <int T> constexpr int ks_max_rows() { return T == kQ6_K ? 2 : 4; }

template <int T>
__device__ __forceinline__ void ks_load(typename KS<T>::Raw &r, const uint8_t *p, int c) {
    if constexpr (T == kQ4_K || T == kQ6_K) KS<T>::load(r, p, c);
    else KS<T>::load(r, p);
}


constexpr int kWaveLdsDwords = 76 * 4;  // per wavefront: 64 uint4 of planes, 16 scales, up to 32 sums

// Workgroup `wg` of a problem: `waves` wavefronts work (threads beyond them only join the final
// barrier); wavefront w handles slices w, w + waves, ... below nslices of the workgroup's 8 * iters rows.
// Those rows are row-steps wg, wg + nwg, wg + 2 nwg, ... of the matrix (nwg: the workgroups of the launch that share it),
// not one block: at any moment the workgroups together read one window of consecutive rows that moves through the
// matrix, as a plain read of the bytes would, instead of nwg streams half a megabyte apart (the seven projections of a
// Llama-3-8B layer in one launch: 22.6 against 23.4 us).  PF divides iters: rows are consumed in groups of PF, buffer j of a
// group always holding the row-step with (it % PF == j).
// WIN <= PF row-steps are kept in flight: WIN go out before the activations are converted, and
// each consumed step is followed by the load of the step WIN ahead, so that load issue (which
// blocks while the memory pipeline is full) and arithmetic alternate instead of forming two
// phases.  Deeper windows lose: on Q4_0 4096 -> 14336 (7 row-steps per wavefront) windows of 3, 4, 5
// and all 7 take 8.0, 8.4, 8.9 and 9.7 us.  (A variant that treats a wavefront's slices x
// row-steps as one sequence, so that the window also spans slices when there are only one or two
// row-steps, was measured: its guarded steps cost the unguarded common case 8 % and it was dropped.)
//
// EXT adds what the callers around a dense layer ask for (fp32 activations only), described by a KsExt:
//   * an RMS normalisation of the activations in front: the gain is multiplied in while a slice
//     is converted, every wavefront adds up the squares of the slices it converts anyway, and
//     the common factor 1 / sqrt(mean(x^2) + eps) - a scalar per activation row - is applied to
//     the finished sums, so the prologue waits for nothing;
//   * a residual added to the result (y may be the residual itself: each output is read and
//     written by one thread);
//   * a second weight matrix W2 (gated feed-forward): the row-steps alternate between W and W2
//     (`iters` counts both and is even), and the result is act(x.W + bias) * (x.W2 + bias2).
struct KsExt {
    const uint8_t *W2;   // second matrix [N, row_bytes], or null
    const float *bias2;  // its bias, or null
    const float *residual;  // added to the result (one value per output), or null
    const float *gain;   // RMS normalisation gain [K], or null for none
    float gain_offset;   // added to every gain
    float eps;
    float inv_k;         // 1 / K
    int norm;            // apply the RMS normalisation
};

//
// R > 1: the pass serves R activation rows at once (xrows <= R of them exist; row r of x lies
// x_stride bytes after row r - 1, of y and of the residual N values): the fixed-point planes of all R
// rows stay in registers and every weight load is contracted against each of them, so a batch of
// two to four rows costs one pass over W, not one per row (the arithmetic stays well below the
// memory time up to four rows).
template <int T, int PF, int WIN, bool EXT = false, bool XBF16 = false, int R = 1, bool PADDED = false>
__device__ __forceinline__ void ks_body(const void *__restrict__ xv, const uint8_t *__restrict__ W,
                                        const float *__restrict__ bias, float *__restrict__ y, int N, int64_t row_bytes, int iters,
                                        int nslices, int half_tail, int act, int waves, int wg, uint32_t *lds, const KsExt *extp = nullptr,
                                        int xrows = 1, int64_t x_stride = 0, int live_iters = 0, int nwg = 1) {
    typedef typename KS<T>::Raw Raw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rg = lane >> 3, c = lane & 7;
    const int rows_wg = iters * 8;
    KsExt ext = {};
    if constexpr (EXT) ext = *extp;
    const bool dual = EXT && ext.W2 != nullptr;
    // PADDED (batched launches, one matrix per problem): the workgroup owns live_iters row-steps of rows; the row-steps from
    // there to `iters` (which the group size divides) read the last of them again - from the caches - and their sums go
    // to slots that are not written out.  So rows per workgroup need not be a multiple of the group size.
    const int live = PADDED ? live_iters : iters;
    float *all = reinterpret_cast<float *>(lds + waves * kWaveLdsDwords);  // partial sums [waves][R][rows_wg]
    float *ssq_w = all + waves * R * rows_wg;                              // EXT: sum of squares [waves][R]
    float ssq[R];
#pragma unroll
    for (int r = 0; r < R; r++) ssq[r] = 0.f;
    // What a lane fetches of slice sl, kept raw until the slice is converted: nothing between the
    // load and the conversion may depend on the loaded values or sit behind a branch, or the
    // wavefront would wait for its activations before it issues the first weight load.  fp32: two
    // float4; bf16: one uint4 (widened at conversion).  The lanes that face the missing half of a
    // last half slice re-read the present half and are zeroed at conversion.
    struct XRaw { uint4 a[R], b[R], ga, gb; bool zero; };
    const bool upper_half = lane >= 32;  // this lane converts values 256 .. 511 of a slice (in both activation layouts)
    const float *gsrc = nullptr;         // EXT: the gain, or any readable stand-in of K floats when there is none
    if constexpr (EXT) gsrc = ext.gain ? ext.gain : reinterpret_cast<const float *>(xv);
    auto x_fetch = [&](int sl) -> XRaw {
        XRaw r;
        r.zero = half_tail && sl == nslices - 1 && upper_half;
        const int xl = r.zero ? lane - 32 : lane;
        r.ga = r.gb = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < R; i++) {  // rows past the last one re-read it (their results are not stored)
            const uint8_t *xrow = reinterpret_cast<const uint8_t *>(xv);
            if constexpr (R > 1) xrow += (int64_t)min(i, xrows - 1) * x_stride;
            r.b[i] = make_uint4(0, 0, 0, 0);
            if constexpr (XBF16) r.a[i] = KS<T>::x_fetch_bf16(reinterpret_cast<const uint16_t *>(xrow) + sl * kSliceValues, xl);
            else KS<T>::x_fetch(reinterpret_cast<const float *>(xrow) + sl * kSliceValues, xl, r.a[i], r.b[i]);
        }
        if constexpr (EXT) {
            // (bf16 activations are half as long as the gain: they cannot stand in for it)
            if (!XBF16 || ext.gain) KS<T>::x_fetch(gsrc + sl * kSliceValues, xl, r.ga, r.gb);
        }
        return r;
    };
    auto as_f4 = [](const uint4 &u) {
        return make_float4(__builtin_bit_cast(float, u.x), __builtin_bit_cast(float, u.y), __builtin_bit_cast(float, u.z),
                           __builtin_bit_cast(float, u.w));
    };
    // the activations a fetched slice stands for (EXT: sum of squares taken, gain applied)
    auto x_values = [&](const XRaw &r, int i) -> XPair {
        XPair p;
        if constexpr (XBF16) p = KS<T>::x_widen_bf16(r.a[i]);
        else { p.lo = as_f4(r.a[i]); p.hi = as_f4(r.b[i]); }
        if (r.zero) { p.lo = make_float4(0.f, 0.f, 0.f, 0.f); p.hi = p.lo; }
        if constexpr (EXT) {
            ssq[i] += (p.lo.x * p.lo.x + p.lo.y * p.lo.y) + (p.lo.z * p.lo.z + p.lo.w * p.lo.w) + (p.hi.x * p.hi.x + p.hi.y * p.hi.y) +
                   (p.hi.z * p.hi.z + p.hi.w * p.hi.w);
            if (ext.gain) {
                const float4 gl = as_f4(r.ga), gh = as_f4(r.gb);
                const float o = ext.gain_offset;
                p.lo.x *= gl.x + o; p.lo.y *= gl.y + o; p.lo.z *= gl.z + o; p.lo.w *= gl.w + o;
                p.hi.x *= gh.x + o; p.hi.y *= gh.y + o; p.hi.z *= gh.z + o; p.hi.w *= gh.w + o;
            }
        }
        return p;
    };
    if (wave < waves) {
        uint4 *my_planes = reinterpret_cast<uint4 *>(lds + wave * kWaveLdsDwords);
        float *my_scales = reinterpret_cast<float *>(my_planes + 64);
        float *my_sums = my_scales + 16;
        float *part = all + wave * R * rows_wg;

        const int spw = (nslices - wave + waves - 1) / waves;  // slices of this wavefront (>= 1)
        XRaw xr = x_fetch(wave);
        const int last_row = N - 1;
        // In a last half slice the lanes of the missing half re-read the codes of the present one
        // (finite scales; their activations are zero).
        auto lane_c = [&](int j) { return (half_tail && wave + j * waves == nslices - 1) ? (c & 3) : c; };
        auto addr = [&](int j, int it) -> const uint8_t * {
            const int step = dual ? it >> 1 : (PADDED ? min(it, live - 1) : it);  // of this workgroup; wg + step * nwg of the matrix
            const int row = min((wg + step * nwg) * 8 + rg, last_row);
            const uint8_t *base = (dual && (it & 1)) ? ext.W2 : W;
            return base + (int64_t)row * row_bytes + (int64_t)(wave + j * waves) * KS<T>::kSliceBytes + KS<T>::lane_offset(lane_c(j));
        };
        Raw buf[PF];
#pragma unroll
        for (int j = 0; j < WIN; j++) ks_load<T>(buf[j], addr(0, j), lane_c(0));

        uint4 xq[R][8];
        constexpr int NS = KS<T>::kScales, SPAN = KS<T>::kSumSpan;
        float xsc[R][NS], xsm[R][NS];
#pragma unroll
        for (int q = 0; q < R; q++)
#pragma unroll
            for (int i = 0; i < NS; i++) xsm[q][i] = 0.f;
        auto stage = [&](const XRaw &r) {
#pragma unroll
            for (int q = 0; q < R; q++) {  // the activation rows take turns in the wavefront's piece of LDS
                const XPair p = x_values(r, q);
                const Staged st = KS<T>::stage(p);
                my_planes[lane] = st.planes;
                if ((lane & 3) == 0) my_scales[lane >> 2] = st.scale;
                if constexpr (SPAN == 32) { if ((lane & 3) == 0) my_sums[lane >> 2] = st.sum; }
                if constexpr (SPAN == 16) { if ((lane & 1) == 0) my_sums[lane >> 1] = st.sum; }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int i = 0; i < 8; i++) xq[q][i] = my_planes[KS<T>::plane_idx(c, i)];
#pragma unroll
                for (int i = 0; i < NS; i++) {
                    xsc[q][i] = my_scales[KS<T>::scale_idx(c, i)];
                    if constexpr (SPAN != 0) xsm[q][i] = my_sums[KS<T>::sum_idx(c, i)];
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        };
        stage(xr);
        if (spw > 1) xr = x_fetch(wave + waves);

        const int ngroups = spw * (iters / PF);
        int j = 0, i0 = 0;  // slice index and first row-step of the current group
        for (int g = 0; g < ngroups; g++) {
            const bool last_group = g == ngroups - 1;
            // where the buffers of this group are refilled from: same slice PF steps on, or the next slice
            const bool wrap = i0 + PF >= iters;
            const int nj = wrap ? j + 1 : j, ni0 = wrap ? 0 : i0 + PF;
#pragma unroll
            for (int jj = 0; jj < PF; jj++) {
                float d[R];
#pragma unroll
                for (int q = 0; q < R; q++) d[q] = KS<T>::dot(buf[jj], xq[q], xsc[q], xsm[q], c);
                if (jj + WIN < PF) ks_load<T>(buf[jj + WIN], addr(j, i0 + jj + WIN), lane_c(j));
                else if (!last_group) ks_load<T>(buf[jj + WIN - PF], addr(nj, ni0 + jj + WIN - PF), lane_c(nj));
#pragma unroll
                for (int q = 0; q < R; q++) {
                    const float t = ks_oct_sum(d[q]);
                    if (c == 0) {
                        float *slot = part + q * rows_wg + (i0 + jj) * 8 + rg;
                        *slot = j == 0 ? t : *slot + t;
                    }
                }
            }
            if (wrap && !last_group) {  // next group starts a new slice: convert its activations
                stage(xr);
                if (nj + 1 < spw) xr = x_fetch(wave + (nj + 1) * waves);
            }
            j = nj;
            i0 = ni0;
        }
        if constexpr (EXT) {
            if (ext.norm) {
#pragma unroll
                for (int q = 0; q < R; q++) {
                    float t = ks_oct_sum(ssq[q]);
                    t += __shfl_xor(t, 8);
                    t += __shfl_xor(t, 16);
                    t += __shfl_xor(t, 32);
                    if (lane == 0) ssq_w[wave * R + q] = t;
                }
            }
        }
    }
    __syncthreads();
    // output row r of activation row q: the wavefronts' partial sums meet here
    const int rows_out = dual ? rows_wg >> 1 : live * 8;
    for (int e = tid; e < rows_out * R; e += blockDim.x) {
        int q = 0, r = e;
        if constexpr (R > 1) { q = e / rows_out; r = e - q * rows_out; }
        const int row = (wg + (r >> 3) * nwg) * 8 + (r & 7);
        if (row >= N) continue;
        if constexpr (R > 1) { if (q >= xrows) continue; }
        const int64_t at = (int64_t)q * N + row;
        if constexpr (EXT) {
            float inv = 1.f;
            if (ext.norm) {
                float t = 0.f;
                for (int w = 0; w < waves; w++) t += ssq_w[w * R + q];
                inv = 1.f / sqrtf(t * ext.inv_k + ext.eps);
            }
            const int slot = dual ? ((r >> 3) * 16 + (r & 7)) : r;  // row-step 2 * (r / 8) of the alternation
            float t = 0.f, u = 0.f;
            for (int w = 0; w < waves; w++) {
                t += all[(w * R + q) * rows_wg + slot];
                if (dual) u += all[(w * R + q) * rows_wg + slot + 8];
            }
            t = apply_act(act, fmaf(t, inv, bias ? bias[row] : 0.f));
            if (dual) t *= fmaf(u, inv, ext.bias2 ? ext.bias2[row] : 0.f);
            if (ext.residual) t += ext.residual[at];
            y[at] = t;
        } else {
            float t = 0.f;
            for (int w = 0; w < waves; w++) t += all[(w * R + q) * rows_wg + r];
            y[at] = apply_act(act, t + (bias ? bias[row] : 0.f));
        }
    }
}

struct KsPlan { int waves, nslices, half_tail, iters, pf, wgs; size_t shmem; };

// GOMLX_HIPQ_GEMV_KS="waves_per_cu" overrides the built-in choice (tuning runs only).
int ks_env_waves() {
    static const int v = [] { const char *e = std::getenv("GOMLX_HIPQ_GEMV_KS"); return e ? std::atoi(e) : 0; }();
    return v;
}

// Slices of 512 values (a last one of 256 when K is an odd multiple of 256) and wavefronts per
// workgroup: one per slice up to 8; more slices than that are dealt out round-robin.
bool ks_split(int64_t K, int &waves, int &nslices, int &half_tail) {
    if (K <= 0 || K % 256 != 0 || K > (int64_t)INT32_MAX / 4) return false;
    nslices = (int)((K + kSliceValues - 1) / kSliceValues);
    half_tail = (K % kSliceValues) != 0 ? 1 : 0;
    waves = nslices < 8 ? nslices : 8;
    return true;
}

size_t ks_lds_bytes(int waves, int iters, int xrows = 1) {  // xrows: activation rows per pass
    return (size_t)waves * kWaveLdsDwords * 4 + (size_t)waves * xrows * iters * 8 * sizeof(float) + 8 * xrows * sizeof(float);  // + sums of squares (EXT)
}

// Row-steps per workgroup and per group: up to 8 row-steps form one group (an even count when two
// matrices alternate); deeper problems run in groups of 4.  (Counts that split into larger equal
// groups, 14 = 2 x 7 instead of 16 = 4 x 4, spread the rows over all workgroups instead of 7/8 of
// them; measured on the gated feed-forward of 2 x 14336 rows it made no difference.  Nor does padding: 14 row-steps per
// workgroup on 256 workgroups, the last group of 4 filled up with re-reads as in the batched launches, took 15.8 against
// 14.8 us for 16 on 224.)
void ks_group(int64_t want, bool even, int &iters, int &pf) {
    if (want < 1) want = 1;
    if (even && (want & 1)) want++;
    if (want <= 8) { iters = pf = (int)want; return; }
    iters = (int)((want + 3) / 4 * 4);
    pf = 4;
}

bool ks_plan(int64_t K, int64_t N, KsPlan &p, bool even_iters = false) {
    if (N <= 0 || !ks_split(K, p.waves, p.nslices, p.half_tail)) return false;
    const int cus = device_cu_count();
    // One 8-wavefront workgroup per CU streams best; problems that would leave a wavefront with
    // only one or two row-steps of a single slice are launch- and latency-bound and get twice the
    // wavefronts (more independent prologues in flight).  Not when a wavefront walks several
    // slices: there two row-steps per slice keep two loads in flight where one row-step keeps
    // one (K = 14336 -> N = 4096: Q4_K 9.9 -> 8.8 us, Q4_0 9.5 -> 8.6, Q6_K 13.2 -> 12.2).
    auto iters_for = [&](int waves_per_cu) {
        int64_t wgs = (int64_t)cus * waves_per_cu / p.waves;
        if (wgs < 1) wgs = 1;
        const int64_t it = (N + wgs * 8 - 1) / (wgs * 8);
        return it < 1 ? (int64_t)1 : it;
    };
    int64_t iters = ks_env_waves() > 0 ? iters_for(ks_env_waves()) : iters_for(8);
    if (ks_env_waves() <= 0 && iters <= 2 && p.nslices <= p.waves) iters = iters_for(16);
    if (iters > kMaxItersKs) iters = kMaxItersKs;
    ks_group(iters, even_iters, p.iters, p.pf);
    p.wgs = (int)((N + (int64_t)p.iters * 8 - 1) / ((int64_t)p.iters * 8));
    p.shmem = ks_lds_bytes(p.waves, p.iters);
    return true;
}

// A plan whose row-steps come in groups of 1, 2 or (if max_pf allows) 4: the multi-row kernels
// exist for those only, and four rows' planes leave registers for two row-steps in flight.
void ks_regroup(KsPlan &p, int64_t N, bool dual, int max_pf) {
    if (p.pf > max_pf || p.pf == 3) {
        p.iters = (p.iters + max_pf - 1) / max_pf * max_pf;
        p.pf = max_pf;
    }
    const int64_t rows_wg = (int64_t)p.iters * (dual ? 4 : 8);
    p.wgs = (int)((N + rows_wg - 1) / rows_wg);
}

// Several independent batch-1 problems of one format in a single launch: workgroups
// [wg_begin, next wg_begin) belong to problem i.  This is how the projections of a decoder layer
// that do not depend on each other (q/k/v, gate/up) share one submission.  Every problem runs in
// groups of two row-steps, both in flight (its iters is a multiple of 2): measured on the seven
// projections of a Llama-3-8B layer, groups of 2 take 23.8 us, 3 / 2 in flight 24.1, 4 / 3 24.7 .. 25.4,
// 8 / 4 25.6 - the finer rounding of rows per workgroup balances the problems better than a deeper
// window helps.  (Measured again with rows per workgroup free of the group size, see PADDED: groups of 4 with 3 in flight
// take 25.0 against 22.8 us: the deeper window itself loses.)
constexpr int kMaxBatchKs = 8;
constexpr int kBatchPF = 2, kBatchWin = 2;
struct KsProblem {
    const float *x;
    const uint8_t *W;
    const float *bias;
    float *y;
    int64_t row_bytes;
    int N, K, iters, live, nslices, half_tail, waves, act, wg_begin, nwg;  // live <= iters row-steps of rows per workgroup, nwg workgroups (see ks_body)
};
struct KsBatch {
    int count;
    KsProblem p[kMaxBatchKs];
};

// Plans one launch for `count` problems (blockIdx.y of the launch walks their activation rows, all of one count): the chip's workgroup slots are shared out in
// proportion to each problem's weight bytes, so every CU streams for about the same time.
template <int T>
int plan_ks_batch(int count, const XsBatchItem *items, KsBatch &b, size_t &shmem, int &wgs) {
    b.count = count;
    const int cus = device_cu_count();
    // A workgroup's time goes with the row-steps of its busiest wavefront: iters x the slices that wavefront walks
    // (more than 8 slices are dealt out round-robin: K = 14336 gives the first four wavefronts 4 slices, the others 3).
    // The smallest common budget of such steps for which all problems together still fit one workgroup per CU decides
    // every problem's rows per workgroup; sharing the CUs out by bytes alone let the problems with uneven slices run a
    // quarter longer than the rest.
    int spw[kMaxBatchKs];  // slices of the busiest wavefront
    for (int i = 0; i < count; i++) {
        KsProblem &q = b.p[i];
        const XsBatchItem &it = items[i];
        q.x = it.x; q.W = it.W; q.bias = it.bias; q.y = it.y; q.N = (int)it.N; q.K = (int)it.K; q.act = it.act;
        q.row_bytes = (int64_t)gq_row_bytes(T, it.K);
        if (!ks_split(it.K, q.waves, q.nslices, q.half_tail)) return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv_ks batch: unsupported K");
        spw[i] = (q.nslices + q.waves - 1) / q.waves;
    }
    // (row-steps of rows per workgroup: any count; the kernel runs them in whole groups of kBatchPF, see live_iters)
    auto iters_for = [&](int i, int budget) {
        int64_t iters = budget / spw[i];
        if (iters < 1) iters = 1;
        if (iters > kMaxItersKs / kBatchPF * kBatchPF) iters = kMaxItersKs / kBatchPF * kBatchPF;
        return iters;
    };
    auto wgs_for = [&](int budget) {
        int64_t n = 0;
        for (int i = 0; i < count; i++) n += (items[i].N + iters_for(i, budget) * 8 - 1) / (iters_for(i, budget) * 8);
        return n;
    };
    int budget = 1;
    const int budget_max = kMaxItersKs * 64;
    while (budget < budget_max && wgs_for(budget) > cus) budget++;
    shmem = 0;
    int wg = 0;
    for (int i = 0; i < count; i++) {
        KsProblem &q = b.p[i];
        const int64_t iters = iters_for(i, budget);
        q.live = (int)iters;
        q.iters = (int)((iters + kBatchPF - 1) / kBatchPF * kBatchPF);
        q.wg_begin = wg;
        wg += (int)((items[i].N + iters * 8 - 1) / (iters * 8));
        q.nwg = wg - q.wg_begin;
        const size_t need = ks_lds_bytes(q.waves, q.iters);
        if (need > shmem) shmem = need;
    }
    wgs = wg;
    return GQ_OK;
}

// the problem that workgroup `wg` of a batched launch belongs to
__device__ __forceinline__ int ks_batch_problem(const KsBatch &b, int wg) {
    int i = 0;
#pragma unroll
    for (int j = 1; j < kMaxBatchKs; j++)
        if (j < b.count && wg >= b.p[j].wg_begin) i = j;
    return i;
}

}  // namespace

}  // namespace gq
