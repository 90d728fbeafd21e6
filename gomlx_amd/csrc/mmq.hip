// Small-batch (decode batch 5..~128; Q4_K up to 512 rows) quantised Dense on the gfx950 matrix cores: Q4_K, and further
// down Q8_0 / Q4_0 / IQ4_NL and Q6_K.
//
// At batch 32 the contraction is 228 flop per weight byte: far beyond the vector ALUs, still
// below the MFMA machine balance, so the kernel should run at the speed the packed weights
// stream from HBM.  Two things decide whether it does:
//
//  * Activation traffic.  Every row tile of W needs all of x.  Fetching x per tile through
//    the CU's vector-memory path would move several times more bytes than the weights themselves, so the
//    work is split along K instead: a workgroup owns a K-slice of up to 7 super-blocks (1792 values; every n-th
//    super-block of a row for n slices, so that the slices' workgroups together read consecutive bytes),
//    keeps the slice of x for 32 batch columns resident in LDS (fp16 in MFMA fragment order, written
//    once by a pre-pass and copied global -> LDS without passing registers) and streams
//    128 rows of W past it.  Slices are summed by a second, tiny kernel that also applies
//    bias and activation (deterministic order, no atomics).
//
//  * VALU work per weight.  Codes are never dequantised to fp32.  A 16-byte run of code bytes
//    becomes four MFMA operand fragments directly in registers: (dword & 0x000F000F) | 0x6400
//    is the fp16 pair (1024 + n_a, 1024 + n_b); one packed fma with the 6-bit sub-block scale
//    gives the exact integers sc*n (<= 945, exact in fp16); these accumulate over a whole
//    super-block on v_mfma_f32_32x32x16_f16, and only then are scaled by the fp16 d in fp32.
//    The sub-block minima (exact 6-bit integers) ride on one extra MFMA per super-block against
//    per-sub-block sums of x, scaled by dmin in fp32.  The only rounding that is not fp32 is x -> fp16 (2^-12 relative).
//
// MFMA roles: A = activations (rows = batch columns), B = weights (columns = W rows), so a
// lane's sixteen results belong to ONE weight row, the one whose header it has already loaded.
#include "blocks.hpp"
#include "common.hpp"

#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace gq {

namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int kSliceSB = 8;                 // super-blocks a slice's activation image has room for (a slice uses up to 7)
constexpr int kSliceK = kSliceSB * 256;     // 2048 values
constexpr int kParts = 2;                   // wavefronts sharing a row tile of 32 (interleaved super-blocks)
constexpr int kMT = 32;                     // batch columns per pass
constexpr int kXFBytes = kSliceK * kMT * 2;          // 131072: fp16 activations, fragment order
constexpr int kXSBytes = kSliceSB * kMT * 16;        // 4096: eight sub-block sums per (super-block, column)
constexpr int kLdsBytes = kXFBytes + kXSBytes;
// Weights are read as consecutive 16-byte chunks of a row (nine per 144-byte super-block, seven rows per load
// instruction) and parked in a wavefront-private piece of LDS, from which lane (row, k-group) picks its header and code
// bytes.  Read one row per lane pair instead (each load instruction touching 32 rows), the same 33 MB of a
// 14336 -> 4096 matrix take 10.9 us against 8.4 us with nothing else going on: the address pattern alone.
constexpr int kParkBytes = 32 * 144;                 // one super-block of a 32-row tile
constexpr int kParkLoads = 5;                        // 288 chunks / 64 lanes
// A workgroup of the Q4_K kernel covers RT row tiles with RT * kParts wavefronts; its LDS holds the slice's image and one
// parked tile per wavefront, which bounds the slice: 7 super-blocks with 4 row tiles (8 wavefronts).  (8 row tiles on 16
// wavefronts with slices of 4 super-blocks, four wavefronts per SIMD and half the image traffic, measured 22.8 us against
// 20.0 us on a 14336 -> 4096 matrix at 32 rows: not built.)
template <int RT> struct Q4KTile {
    static_assert(RT == 4, "LDS budget below is for four row tiles");
    static constexpr int kWaves = RT * kParts, kRows = 32 * RT;
    static constexpr int kMaxSliceSB = 7;
    static constexpr int kLds = kMaxSliceSB * 16384 + kXSBytes + kWaves * kParkBytes;
    static_assert(kLds <= 160 * 1024, "image + parked tiles exceed LDS");
};
constexpr int kQ4KRowTiles = 4;

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    h2 v;
    v.x = (_Float16)a;
    v.y = (_Float16)b;
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }

// Eight consecutive activations as fp32: from fp32 memory, or from bf16 memory widened (exact).
template <bool BF16X>
__device__ __forceinline__ void load_x8(const void *X, int64_t index, float4 &lo, float4 &hi) {
    if constexpr (BF16X) {
        const uint4 v = *reinterpret_cast<const uint4 *>(static_cast<const uint16_t *>(X) + index);
        lo = make_float4(__builtin_bit_cast(float, v.x << 16), __builtin_bit_cast(float, v.x & 0xFFFF0000u),
                         __builtin_bit_cast(float, v.y << 16), __builtin_bit_cast(float, v.y & 0xFFFF0000u));
        hi = make_float4(__builtin_bit_cast(float, v.z << 16), __builtin_bit_cast(float, v.z & 0xFFFF0000u),
                         __builtin_bit_cast(float, v.w << 16), __builtin_bit_cast(float, v.w & 0xFFFF0000u));
    } else {
        const float4 *p = reinterpret_cast<const float4 *>(static_cast<const float *>(X) + index);
        lo = p[0];
        hi = p[1];
    }
}

// (u & mask) | 0x64006400 as an fp16 pair: 1024 + n (mask 0x000F000F), 1024 + 16 n (0x00F000F0)
// or 1024 + byte (0x00FF00FF)
// The 0x64006400 operand is passed in a register: with two literals the compiler has to split the
// operation into v_and + v_or, with one it is a single v_and_or_b32.
__device__ __forceinline__ h2 magic_pair(uint32_t u, uint32_t mask, uint32_t magic) { return as_h2((u & mask) | magic); }

__device__ __forceinline__ float dpp_quad_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    return v;
}

// RMS normalisation folded into the split-K route: the pre-pass multiplies x by (gain + offset) before it scales and
// rounds, and leaves each (slice, column)'s sum of squares of the raw x in xss[slice][M]; the reduction divides the
// finished sums of column m by sqrt(sum_s xss[s][m] / K + eps) (the contraction is linear in x).
__device__ __forceinline__ float sumsq8(const float4 &a, const float4 &b) {
    return ((a.x * a.x + a.y * a.y) + (a.z * a.z + a.w * a.w)) + ((b.x * b.x + b.y * b.y) + (b.z * b.z + b.w * b.w));
}
__device__ __forceinline__ void apply_gain8(const float *__restrict__ gain, float off, int k, float4 &a, float4 &b) {  // gain 16-byte aligned, k % 8 == 0
    const float4 g0 = *reinterpret_cast<const float4 *>(gain + k), g1 = *reinterpret_cast<const float4 *>(gain + k + 4);
    a.x *= g0.x + off; a.y *= g0.y + off; a.z *= g0.z + off; a.w *= g0.w + off;
    b.x *= g1.x + off; b.y *= g1.y + off; b.z *= g1.z + off; b.w *= g1.w + off;
}
__device__ __forceinline__ float wave_sum(float v) {
    for (int m = 1; m < 64; m <<= 1) v += __shfl_xor(v, m);
    return v;
}

// ---- stage the K-slice of x into LDS in MFMA fragment order ---------------------------------
//
// One item = 8 consecutive activations of one batch column ("octet").  Inside a super-block the
// value index v = 64 g' + 32 high + idx: byte idx of group g', low (high = 0) or high nibble.
// The main loop loads the 16-byte chunk c = 2 g' + idx / 16 and turns it into four octets
// q = 2 high + (idx % 16) / 8, the code bytes inside an octet coming out in the order
// (0, 2, 1, 3, 4, 6, 5, 7).  Octet (sbl, c, q) of column m lives in slot (8 sbl + c) * 4 + q at
// column position m ^ (slot & 15): consecutive threads hold consecutive octets of ONE column,
// i.e. different slots with the same m, and the xor spreads their 16-byte stores (and the 32
// columns a half-wave later reads from one slot) over all LDS banks.
// The eight sub-block sums of (sbl, m) are stored in the order (0, 2, 1, 3, 4, 6, 5, 7) too.
// `active`: the thread's octet belongs to the slice (slices may hold fewer than 8 super-blocks).
// red: [2][2][ROUNDS][4] floats of shared memory; inv_scale[m] receives the slice's inverse scale of column m0 + m.
// With xss (normalisation folded in): x is multiplied by gain + gain_offset (gain may be null) and xss[m0 + m] receives
// the slice's sum of squares of the raw x.
template <int ROUNDS, bool BF16X>
__device__ __forceinline__ void stage_x(const void *__restrict__ X, int M, int K, int m0, int sb_first, int sb_stride, uint8_t *__restrict__ lds, int tid,
                                        int round0, bool active, float *red, float *__restrict__ inv_scale, const float *__restrict__ gain,
                                        float gain_offset, float *__restrict__ xss) {
    const int oct = tid & 255;  // fixed per thread; its items are columns (tid >> 8) + 2 r
    const int k = ((oct >> 5) * sb_stride + sb_first) * 256 + 8 * (oct & 31);  // super-block sbl of the slice is sb_first + sbl * sb_stride of the row
    const int sbl = oct >> 5, v8 = oct & 31;
    const int gp = v8 >> 3, w8 = v8 & 7, high = w8 >> 2, idx8 = w8 & 3;
    const int q = high * 2 + (idx8 & 1), c = 2 * gp + (idx8 >> 1);
    const int slot = (sbl * 8 + c) * 4 + q, swz = slot & 15;
    const int j = 2 * gp + high;
    const int jpos = (j & 4) | ((j & 1) << 1) | ((j >> 1) & 1);
    uint8_t *xf_base = lds + slot * (kMT * 16);
    uint8_t *xs_base = lds + kXFBytes + sbl * (kMT * 16) + jpos * 2;
    const bool k_ok = active && k < K;
    const int ksrc = max(min(k, K - 8), 0);
    float4 lo[ROUNDS], hi[ROUNDS];
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) {
        const int m = (tid >> 8) + 2 * (round0 + r);
        load_x8<BF16X>(X, (int64_t)min(m0 + m, M - 1) * K + ksrc, lo[r], hi[r]);
    }
    // largest magnitude of each column's slice: its 256 octets sit in the four wavefronts of one half of the workgroup
    const int half = tid >> 8, wih = (tid >> 6) & 3;
    float *red_ss = red + 2 * ROUNDS * 4;
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) {
        const bool ok = k_ok && (m0 + half + 2 * (round0 + r) < M);
        if (xss) {
            const float ss = wave_sum(ok ? sumsq8(lo[r], hi[r]) : 0.f);
            if ((tid & 63) == 0) red_ss[(half * ROUNDS + r) * 4 + wih] = ss;
            if (gain) apply_gain8(gain, gain_offset, ksrc, lo[r], hi[r]);
        }
        const float am = wave_max(ok ? amax8(lo[r], hi[r]) : 0.f);
        if ((tid & 63) == 0) red[(half * ROUNDS + r) * 4 + wih] = am;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) {
        const int m = (tid >> 8) + 2 * (round0 + r);
        const bool ok = k_ok && (m0 + m < M);
        const float *rr = red + (half * ROUNDS + r) * 4;
        float sc, inv;
        pow2_scale(fmaxf(fmaxf(rr[0], rr[1]), fmaxf(rr[2], rr[3])), sc, inv);
        if (oct == 0 && m0 + m < M) {
            inv_scale[m0 + m] = inv;
            if (xss) {
                const float *rs = red_ss + (half * ROUNDS + r) * 4;
                xss[m0 + m] = (rs[0] + rs[1]) + (rs[2] + rs[3]);
            }
        }
        if (!active) continue;
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        float4 a = ok ? lo[r] : z, b = ok ? hi[r] : z;
        a.x *= sc; a.y *= sc; a.z *= sc; a.w *= sc; b.x *= sc; b.y *= sc; b.z *= sc; b.w *= sc;
        uint4 o;  // bytes (0,2,1,3,4,6,5,7)
        o.x = pack_h2(a.x, a.z);
        o.y = pack_h2(a.y, a.w);
        o.z = pack_h2(b.x, b.z);
        o.w = pack_h2(b.y, b.w);
        *reinterpret_cast<uint4 *>(xf_base + (m ^ swz) * 16) = o;
        float sum = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w));
        sum = dpp_quad_sum(sum);  // the four octets of one 32-value sub-block sit in one quad
        if (idx8 == 0) *reinterpret_cast<_Float16 *>(xs_base + m * 16) = (_Float16)sum;
    }
}

struct RawSB { uint4 hd, c[4]; };  // header + this lane's four chunks (steps 0..3)



// One super-block of a 32-row tile against the staged activations: `cur` is lane (row col, k-group kg)'s header and code
// bytes, `lds` the fragment image (slot-major, see stage_x), `sums` the sub-block sums of the super-block's 32 columns
// (16 bytes each).  SBSCALE: the activations of this super-block carry their own power-of-two scale per column, whose
// inverses (`inv`, 32 floats) multiply the block's contribution; otherwise the caller's slice-wide scale is applied later.
template <bool SBSCALE>
__device__ __forceinline__ void q4k_contract_sb(const RawSB &cur, const uint8_t *lds, const uint8_t *sums, const float *inv, int sbl, int kg, int col,
                                                uint32_t magic, f16v &acc) {
    const float d = half_bits_to_float(cur.hd.x & 0xFFFFu), dmin = half_bits_to_float(cur.hd.x >> 16);
    // all eight 6-bit scales / minima as bytes: sc0..3, sc4..7, m0..3, m4..7
    const uint32_t a = cur.hd.y, b = cur.hd.z, c = cur.hd.w;
    const uint32_t sc_lo = a & 0x3F3F3F3Fu, mn_lo = b & 0x3F3F3F3Fu;
    const uint32_t sc_hi = (c & 0x0F0F0F0Fu) | ((a >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((c >> 4) & 0x0F0F0F0Fu) | ((b >> 2) & 0x30303030u);
    f16v p1;
#pragma unroll
    for (int r = 0; r < 16; r++) p1[r] = 0.f;
    // all sixteen activation fragments of this super-block are requested up front so that the
    // LDS latency hides behind the code conversion below
    h8 xfr[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int slot = (sbl * 8 + 2 * (i >> 2) + kg) * 4 + (i & 3);
        xfr[i] = *reinterpret_cast<const h8 *>(lds + (slot * kMT + (col ^ (slot & 15))) * 16);
    }
#pragma unroll
    for (int st = 0; st < 4; st++) {
        // chunk 2 st + kg lies in group st: sub-block 2 st in the low nibbles, 2 st + 1 in the high ones
        const uint32_t scw = (st < 2 ? sc_lo : sc_hi) >> (16 * (st & 1));
        const float s0f = (float)(scw & 0xFFu), s1f = (float)((scw >> 8) & 0xFFu);
        const h2 s0 = as_h2(pack_h2(s0f, s0f));
        const h2 s1 = as_h2(pack_h2(s1f * 0.0625f, s1f * 0.0625f));  // high-nibble pairs arrive as 1024 + 16 n
        const h2 k0h = as_h2(pack_h2(-1024.f * s0f, -1024.f * s0f));
        const h2 k1h = as_h2(pack_h2(-64.f * s1f, -64.f * s1f));
        const uint32_t dw[4] = {cur.c[st].x, cur.c[st].y, cur.c[st].z, cur.c[st].w};
        uint32_t wl[8], wh[8];
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t u = dw[w], v = dw[w] >> 8;
            wl[2 * w] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(u, 0x000F000Fu, magic), s0, k0h));
            wl[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(v, 0x000F000Fu, magic), s0, k0h));
            wh[2 * w] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(u, 0x00F000F0u, magic), s1, k1h));
            wh[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(v, 0x00F000F0u, magic), s1, k1h));
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t *src = (q < 2 ? wl : wh) + 4 * (q & 1);
            const h8 wfrag = __builtin_bit_cast(h8, make_uint4(src[0], src[1], src[2], src[3]));
            p1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(xfr[4 * st + q], wfrag, p1, 0, 0, 0);
        }
    }
    // minima: k-group 0 carries the exact integers (m0, m2, m1, m3, m4, m6, m5, m7) against the sub-block sums of x in
    // the same order; dmin multiplies the finished fp32 sums below, as d multiplies p1 (in an fp16 operand dmin * m
    // would be rounded to 11 bits, and overflow from dmin = 1040 on)
    f16v p2, zero16;
#pragma unroll
    for (int r = 0; r < 16; r++) zero16[r] = 0.f;
    {
        uint4 mv = make_uint4(0u, 0u, 0u, 0u), sv = make_uint4(0u, 0u, 0u, 0u);
        if (kg == 0) {
            const h2 off = as_h2(0xE400E400u);  // (-1024, -1024)
            mv.x = __builtin_bit_cast(uint32_t, magic_pair(mn_lo, 0x00FF00FFu, magic) + off);
            mv.y = __builtin_bit_cast(uint32_t, magic_pair(mn_lo >> 8, 0x00FF00FFu, magic) + off);
            mv.z = __builtin_bit_cast(uint32_t, magic_pair(mn_hi, 0x00FF00FFu, magic) + off);
            mv.w = __builtin_bit_cast(uint32_t, magic_pair(mn_hi >> 8, 0x00FF00FFu, magic) + off);
            sv = *reinterpret_cast<const uint4 *>(sums + col * 16);
        }
        p2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, sv), __builtin_bit_cast(h8, mv), zero16, 0, 0, 0);
    }
    if constexpr (SBSCALE) {
        // lane holds columns m = 8 (r / 4) + 4 kg + r % 4
        float4 iv[4];
#pragma unroll
        for (int g = 0; g < 4; g++) iv[g] = reinterpret_cast<const float4 *>(inv)[2 * g + kg];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float f = (r & 3) == 0 ? iv[r >> 2].x : (r & 3) == 1 ? iv[r >> 2].y : (r & 3) == 2 ? iv[r >> 2].z : iv[r >> 2].w;
            acc[r] = fmaf(f, fmaf(-dmin, p2[r], d * p1[r]), acc[r]);
        }
    } else {
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = fmaf(d, p1[r], acc[r]);
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = fmaf(-dmin, p2[r], acc[r]);
    }
}

// One super-block against the images of RM tiles of 32 batch columns at once: the codes are turned into operand fragments
// ONCE and every fragment meets each tile's activations, so the conversion, the parked tile and the header are shared by
// up to 128 batch rows.  Per tile the arithmetic and its order are those of q4k_contract_sb<false>.  The work comes in two
// halves (steps 2 H and 2 H + 1 of the super-block's four), so that the images can be staged half a super-block at a time:
// `img` holds tile t's half at 8192 t - 16 slots of (32 columns x 16 bytes) in the order of stage_x, whose slot index
// modulo 16 is the position inside the half.
template <int RM, int H>
__device__ __forceinline__ void q4k_tiles_half(const RawSB &cur, const uint8_t *img, int kg, int col, uint32_t magic, f16v (&p1)[RM]) {
    const uint32_t a = cur.hd.y, c = cur.hd.w;
    const uint32_t sc = H == 0 ? (a & 0x3F3F3F3Fu) : ((c & 0x0F0F0F0Fu) | ((a >> 2) & 0x30303030u));  // scales 0..3 / 4..7 as bytes
    // Eight groups (step s2, fragment q) of RM MFMAs each; the activations of group g + 1 are requested from LDS before the
    // MFMAs of group g are issued and nothing moves across the group boundaries, so that two groups' fragments are all the
    // registers the reads take (left to itself the compiler hoists sixteen reads and more, and four tiles spill).
    h8 xf[2][RM];
    auto request = [&](int g) __attribute__((always_inline)) {
        const int slot = (2 * (g >> 2) + kg) * 4 + (g & 3);  // fragment 4 st + q sits in slot 32 sb + 8 st + 4 kg + q of the image: this is that modulo 16
#pragma unroll
        for (int t = 0; t < RM; t++) xf[g & 1][t] = *reinterpret_cast<const h8 *>(img + t * 8192 + (slot * kMT + (col ^ slot)) * 16);
    };
    request(0);
    uint32_t wl[8], wh[8];
#pragma unroll
    for (int g = 0; g < 8; g++) {
        const int s2 = g >> 2, q = g & 3;
        if (q == 0) {
            const int st = 2 * H + s2;
            const uint32_t scw = sc >> (16 * s2);
            const float s0f = (float)(scw & 0xFFu), s1f = (float)((scw >> 8) & 0xFFu);
            const h2 s0 = as_h2(pack_h2(s0f, s0f));
            const h2 s1 = as_h2(pack_h2(s1f * 0.0625f, s1f * 0.0625f));  // high-nibble pairs arrive as 1024 + 16 n
            const h2 k0h = as_h2(pack_h2(-1024.f * s0f, -1024.f * s0f));
            const h2 k1h = as_h2(pack_h2(-64.f * s1f, -64.f * s1f));
            const uint32_t dw[4] = {cur.c[st].x, cur.c[st].y, cur.c[st].z, cur.c[st].w};
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t u = dw[w], v = dw[w] >> 8;
                wl[2 * w] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(u, 0x000F000Fu, magic), s0, k0h));
                wl[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(v, 0x000F000Fu, magic), s0, k0h));
                wh[2 * w] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(u, 0x00F000F0u, magic), s1, k1h));
                wh[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(v, 0x00F000F0u, magic), s1, k1h));
            }
        }
        if (g + 1 < 8) request(g + 1);
        const uint32_t *src = (q < 2 ? wl : wh) + 4 * (q & 1);
        const h8 wfrag = __builtin_bit_cast(h8, make_uint4(src[0], src[1], src[2], src[3]));
#pragma unroll
        for (int t = 0; t < RM; t++) p1[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xf[g & 1][t], wfrag, p1[t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The end of a super-block: the minima against the tiles' sub-block sums (tile t's at sums + 1024 t), then d and dmin in fp32;
// p1 starts the next super-block at zero.  Only k-group 0 carries operands of the minima's MFMA (the sums are read by
// every lane and cleared by a mask in k-group 1: no branch around an LDS read).
template <int RM>
__device__ __forceinline__ void q4k_tiles_finish(const RawSB &cur, const uint8_t *sums, int kg, int col, uint32_t magic, f16v (&p1)[RM], f16v (&acc)[RM]) {
    const float d = half_bits_to_float(cur.hd.x & 0xFFFFu), dmin = half_bits_to_float(cur.hd.x >> 16);
    const uint32_t a = cur.hd.y, b = cur.hd.z, c = cur.hd.w;
    (void)a;
    const uint32_t mn_lo = b & 0x3F3F3F3Fu, mn_hi = ((c >> 4) & 0x0F0F0F0Fu) | ((b >> 2) & 0x30303030u);
    f16v zero16;
#pragma unroll
    for (int r = 0; r < 16; r++) zero16[r] = 0.f;
    const uint32_t keep = kg == 0 ? 0xFFFFFFFFu : 0u;
    const h2 off = as_h2(0xE400E400u);  // (-1024, -1024)
    uint4 mv;
    mv.x = __builtin_bit_cast(uint32_t, magic_pair(mn_lo, 0x00FF00FFu, magic) + off) & keep;
    mv.y = __builtin_bit_cast(uint32_t, magic_pair(mn_lo >> 8, 0x00FF00FFu, magic) + off) & keep;
    mv.z = __builtin_bit_cast(uint32_t, magic_pair(mn_hi, 0x00FF00FFu, magic) + off) & keep;
    mv.w = __builtin_bit_cast(uint32_t, magic_pair(mn_hi >> 8, 0x00FF00FFu, magic) + off) & keep;
#pragma unroll
    for (int t = 0; t < RM; t++) {
        // (a native vector type: read as HIP's uint4 struct the load loses what tells the compiler that it cannot touch the
        // destination of a load into LDS, and it then waits for every such load in flight before this read)
        typedef uint32_t Quad __attribute__((ext_vector_type(4)));
        Quad sv = *reinterpret_cast<const Quad *>(sums + t * 1024 + col * 16);
        sv &= keep;
        const f16v p2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, sv), __builtin_bit_cast(h8, mv), zero16, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 16; r++) acc[t][r] = fmaf(d, p1[t][r], acc[t][r]);
#pragma unroll
        for (int r = 0; r < 16; r++) acc[t][r] = fmaf(-dmin, p2[r], acc[t][r]);
#pragma unroll
        for (int r = 0; r < 16; r++) p1[t][r] = 0.f;
    }
}

// Activation pre-pass: writes each (K-slice, column tile)'s LDS image (fragment-ordered fp16
// activations + sub-block sums) to global memory once; the row-range workgroups of the main
// kernel then only copy 132 KiB each instead of converting it again.  grid = (slices, column
// tiles, 8): each workgroup converts four of the tile's 32 columns.
// slice_sb <= 8 super-blocks per slice: a thread whose octet lies beyond them has nothing to do (the
// image keeps its 8-super-block layout; the main kernel copies and uses the first slice_sb only).
// xscale[slice][M]: the inverse of the power of two that (slice, column) was scaled by.
template <bool BF16X, int ROUNDS>
__global__ __launch_bounds__(512) void mmq_xprep_kernel(const void *__restrict__ X, uint8_t *__restrict__ ximg, float *__restrict__ xscale, int M,
                                                        int K, int slice_sb, const float *__restrict__ gain, float gain_offset,
                                                        float *__restrict__ xss) {
    __shared__ float red[2 * 2 * ROUNDS * 4];
    const int slice = blockIdx.x, mt = blockIdx.y;
    const bool active = (((int)threadIdx.x & 255) >> 5) < slice_sb;
    stage_x<ROUNDS, BF16X>(X, M, K, mt * kMT, slice, (int)gridDim.x, ximg + ((size_t)mt * gridDim.x + slice) * kLdsBytes, threadIdx.x,
                      ROUNDS * blockIdx.z, active, red, xscale + (size_t)slice * M, gain, gain_offset, xss ? xss + (size_t)slice * M : nullptr);
}

// Up to four matrices that are contracted against one activation image in one launch (the q / k / v projections behind
// one normalisation): matrix p owns workgroups wg0[p] .. of grid.x and columns n0[p] .. n0[p] + N[p] - 1 of the
// partial sums, whose rows are ntot = sum of N[p] long.
constexpr int kMaxSet = 4;
struct Q4KSet {
    const uint8_t *W[kMaxSet];
    int N[kMaxSet], wg0[kMaxSet], n0[kMaxSet];
    int count, ntot;
};

// partial[slice][m][n0[p] + n] = sum over the slice's k of x[m][k] * w_p[n][k]
//
// RT * kParts wavefronts: wavefront w contracts row tile w % RT (32 rows of W) over the
// super-blocks w / RT, w / RT + kParts, ... of the slice; the partial tiles meet in LDS at the end.  v_mfma_f32_32x32x16_f16 with
// A = activations (32 batch columns x 16 k) and B = weights (16 k x 32 rows): one 16-byte LDS
// read per lane feeds 16384 multiply-adds, and a lane's 16 results all belong to its own row.
template <int RT>
__global__ __launch_bounds__(64 * RT * kParts) void mmq_q4k_kernel(const uint8_t *__restrict__ ximg, Q4KSet set,
                                                      float *__restrict__ partial0, int M, int K,
                                                      int64_t row_bytes, int m0, int slice_sb, const uint8_t *__restrict__ W2,
                                                      float *__restrict__ partial2) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // blockIdx.z = 1: the second matrix of a gated pair (same activation image, its own partial sums)
    int prob = 0;
#pragma unroll
    for (int j = 1; j < kMaxSet; j++)
        if (j < set.count && (int)blockIdx.x >= set.wg0[j]) prob = j;
    const uint8_t *__restrict__ W = blockIdx.z ? W2 : set.W[prob];
    float *__restrict__ partial = blockIdx.z ? partial2 : partial0;
    const int N = set.N[prob], xblk = (int)blockIdx.x - set.wg0[prob];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 5, col = lane & 31;
    const int rt = wave % RT, par = wave / RT;  // par = 0 .. kParts-1
    const int slice = blockIdx.y;
    // Slice s holds super-blocks s, s + nslices, s + 2 nslices, ... of every row: the workgroups of a row range, which
    // run side by side, then read one stretch of consecutive bytes of each row at a time and move along the rows together.
    const int nslices = gridDim.y;
    const int nsb = ((K >> 8) - slice + nslices - 1) / nslices;
    const int n = xblk * (32 * RT) + rt * 32 + col;  // this lane's weight row

    // the slice's activation image goes straight from global memory into LDS (no registers)
    {
        const uint8_t *img = ximg + ((size_t)(m0 / kMT) * gridDim.y + slice) * kLdsBytes;
        // fragments of the slice's first slice_sb super-blocks (16 KiB each), then the 4 KiB of sub-block sums
        const int frag_kib = slice_sb * 16;
        for (int i0 = wave; i0 < frag_kib + kXSBytes / 1024; i0 += RT * kParts) {
            const int i = i0 < frag_kib ? i0 : kXFBytes / 1024 + (i0 - frag_kib);
            // (in LDS the sums follow the fragments directly; the image in memory keeps room for 8 super-blocks)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(img + i * 1024 + lane * 16),
                                             (__attribute__((address_space(3))) void *)(lds + i0 * 1024), 16, 0, 0);
        }
    }
    const int xs_off = slice_sb * 16384;
    // Chunk c = lane + 64 l of a (32 rows x 144 bytes) tile is piece c % 9 of row c / 9.  The chunks go from global
    // memory straight into the wavefront's piece of LDS (no registers held while they are in flight): each load
    // instruction writes 64 lanes x 16 bytes to consecutive LDS addresses, which is the tile's own layout.
    // (byte offsets from the first row of the tile: mmq_supported keeps 31 rows below 2^32 bytes)
    const int row0 = xblk * (32 * RT) + rt * 32;
    const uint8_t *wtile = W + (int64_t)min(row0, N - 1) * row_bytes + slice * 144;
    uint32_t csrc[kParkLoads];
#pragma unroll
    for (int l = 0; l < kParkLoads; l++) {
        const int c = min(lane + 64 * l, 32 * 9 - 1);
        csrc[l] = (uint32_t)(min(row0 + c / 9, N - 1) - min(row0, N - 1)) * (uint32_t)row_bytes + (uint32_t)((c % 9) * 16);
    }
    uint8_t *park = lds + xs_off + kXSBytes + wave * kParkBytes;
    auto fetch = [&](int sb) __attribute__((always_inline)) {
        const uint8_t *base = wtile + sb * nslices * 144;
#pragma unroll
        for (int l = 0; l < kParkLoads; l++)
            if (64 * l + 64 <= 32 * 9 || lane < 32 * 9 - 64 * l)  // (the last instruction carries 32 chunks)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(base + csrc[l]),
                                                 (__attribute__((address_space(3))) void *)(park + l * 1024), 16, 0, 0);
    };
    if (par < nsb) fetch(par);
    const uint8_t *myrow = park + col * 144;
    // a barrier does not wait for loads in flight: every wavefront's share of the image copy must have landed in LDS
    // before it arrives (the wait also covers the wavefront's own first tile, which the loop would wait for next anyway)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    f16v acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));

    for (int sbl = par; sbl < nsb; sbl += kParts) {
        // the tile's super-block has landed in this wavefront's piece of LDS: pick out this lane's part, and once those
        // reads are done request the next super-block into the same place
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        typedef uint32_t Chunk __attribute__((ext_vector_type(4)));
        Chunk rhd = *reinterpret_cast<const Chunk *>(myrow), rc[4];
#pragma unroll
        for (int st = 0; st < 4; st++) rc[st] = *reinterpret_cast<const Chunk *>(myrow + 16 + 32 * st + 16 * kg);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(rhd), "+v"(rc[0]), "+v"(rc[1]), "+v"(rc[2]), "+v"(rc[3])::"memory");
        RawSB cur;
        cur.hd = make_uint4(rhd.x, rhd.y, rhd.z, rhd.w);
#pragma unroll
        for (int st = 0; st < 4; st++) cur.c[st] = make_uint4(rc[st].x, rc[st].y, rc[st].z, rc[st].w);
        __builtin_amdgcn_wave_barrier();
        if (sbl + kParts < nsb) fetch(sbl + kParts);
        q4k_contract_sb<false>(cur, lds, lds + xs_off + sbl * (kMT * 16), nullptr, sbl, kg, col, magic, acc);
    }

    // wavefronts 1..kParts-1 of a row tile hand their 32 x 32 partial tiles to wavefront 0 through LDS
    __syncthreads();
    float *xch = reinterpret_cast<float *>(lds) + rt * ((kParts - 1) * 16 * 64);
    if (par > 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) xch[((par - 1) * 16 + r) * 64 + lane] = acc[r];
    }
    __syncthreads();
    if (par == 0 && n < N) {
        // lane holds y[m = 8 (r / 4) + 4 kg + r % 4][n] for its K-slice
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = m0 + 8 * (r >> 2) + 4 * kg + (r & 3);
            float v = acc[r];
#pragma unroll
            for (int p = 0; p < kParts - 1; p++) v += xch[(p * 16 + r) * 64 + lane];
            if (m < M) partial[((int64_t)slice * M + m) * set.ntot + set.n0[prob] + n] = v;
        }
    }
}

// ---- several tiles of 32 batch rows per weight tile ---------------------------------------------------------------
//
// mmq_q4k_kernel serves one tile of 32 batch rows per launch: 128 rows stream W four times and convert every code four
// times.  mmq_q4k_tiles_kernel walks up to four such tiles together: eight wavefronts, each with its own row tile of 32 rows
// of W (256 per workgroup) and all of the slice's super-blocks.  The activation images of four tiles do not fit LDS for a
// whole slice, so the workgroup moves along K half a super-block at a time: the halves of every tile's image (8 KiB each,
// global -> LDS by DMA from the pre-pass's image) go through a ring of two stages - while the wavefronts contract one
// half (q4k_tiles_half: every converted fragment against all tiles), the next is on its way - with one barrier per half.
// A wavefront's weight tiles are parked two super-blocks ahead.  The waits are counted: a wavefront's loads complete in
// the order they were issued, so "at most five outstanding" after a request of a weight tile (five load instructions)
// means that everything older has landed, the image half among it.
// Same grid roles, same image and partial-sum layouts as mmq_q4k_kernel (m0 = first batch row, NT = tiles of 32 from there).
struct Q4KTiles {
    static constexpr int kMaxTiles = 4, kWaves = 8, kRows = 32 * kWaves;
    static constexpr int kHalfBytes = 8192;                                    // half a super-block of one tile's image
};
// LDS of the kernel for NT tiles: [ring: 2 stages x NT halves][sums][parked weight tiles].  A single tile keeps one parked
// tile per wavefront, which lets two workgroups share a CU (53 KiB each); more tiles are bound to one workgroup by their
// registers anyway and park two.
template <int NT> struct Q4KTilesOf {
    static constexpr int kStageBytes = NT * Q4KTiles::kHalfBytes;
    static constexpr int kRingBytes = 2 * kStageBytes;
    static constexpr int kSumBytes = NT * 1024;                                // sub-block sums of one super-block: 512 bytes per tile, 1 KiB apart
    static constexpr int kParks = NT == 1 ? 1 : 2;                             // weight tiles on their way per wavefront
    static constexpr int kLds = kRingBytes + kSumBytes + kParks * Q4KTiles::kWaves * kParkBytes;
    static_assert(kLds <= 160 * 1024, "images + parked tiles exceed LDS");
};

template <int NT>
__global__ __launch_bounds__(64 * Q4KTiles::kWaves) void mmq_q4k_tiles_kernel(const uint8_t *__restrict__ ximg, Q4KSet set, float *__restrict__ partial0,
                                                                               int M, int K, int64_t row_bytes, int m0,
                                                                               const uint8_t *__restrict__ W2, float *__restrict__ partial2) {
    typedef Q4KTiles G;
    typedef Q4KTilesOf<NT> L;
    static_assert(NT >= 1 && NT <= G::kMaxTiles, "one to four tiles of 32 batch rows");
    static_assert(kParkLoads == 5, "the counted waits below assume five load instructions per weight tile");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    int prob = 0;
#pragma unroll
    for (int j = 1; j < kMaxSet; j++)
        if (j < set.count && (int)blockIdx.x >= set.wg0[j]) prob = j;
    const uint8_t *__restrict__ W = blockIdx.z ? W2 : set.W[prob];
    float *__restrict__ partial = blockIdx.z ? partial2 : partial0;
    const int N = set.N[prob], xblk = (int)blockIdx.x - set.wg0[prob];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 5, col = lane & 31;
    const int slice = blockIdx.y, nslices = gridDim.y;
    const int nsb = ((K >> 8) - slice + nslices - 1) / nslices;  // slice s holds super-blocks s, s + nslices, ... of every row (at least one)
    const int row0 = xblk * G::kRows + wave * 32;
    const int n = row0 + col;  // this lane's weight row

    const uint8_t *wtile = W + (int64_t)min(row0, N - 1) * row_bytes + slice * 144;
    uint32_t csrc[kParkLoads];
#pragma unroll
    for (int l = 0; l < kParkLoads; l++) {
        const int c = min(lane + 64 * l, 32 * 9 - 1);
        csrc[l] = (uint32_t)(min(row0 + c / 9, N - 1) - min(row0, N - 1)) * (uint32_t)row_bytes + (uint32_t)((c % 9) * 16);
    }
    uint8_t *const park0 = lds + L::kRingBytes + L::kSumBytes + wave * (L::kParks * kParkBytes);
    // super-block j of this wavefront's row tile -> park j % kParks: exactly kParkLoads load instructions
    auto fetch = [&](int sb) __attribute__((always_inline)) {
        const uint8_t *base = wtile + sb * nslices * 144;
        uint8_t *park = park0 + (sb % L::kParks) * kParkBytes;
#pragma unroll
        for (int l = 0; l < kParkLoads; l++)
            if (64 * l + 64 <= 32 * 9 || lane < 32 * 9 - 64 * l)  // (the last instruction carries 32 chunks)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(base + csrc[l]),
                                                 (__attribute__((address_space(3))) void *)(park + l * 1024), 16, 0, 0);
    };
    // tile t's image of this slice: fragments of super-block j at 16384 j (its second half 8192 further), sums at kXFBytes + 512 j
    const uint8_t *img0 = ximg + ((size_t)(m0 / kMT) * nslices + slice) * kLdsBytes;
    const size_t tile_stride = (size_t)nslices * kLdsBytes;
    // half `h` of super-block `sb` of every tile -> ring stage h; with the second half come the super-block's sub-block sums, which
    // are read at its end and not again (one buffer, at a fixed address: the compiler's own wait insertion can tell it from the ring)
    auto stage = [&](int sb, int h) __attribute__((always_inline)) {
        uint8_t *dst = lds + h * L::kStageBytes;
        for (int i = wave; i < NT * 8; i += G::kWaves) {
            const int t = i >> 3, ck = i & 7;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void *)(img0 + t * tile_stride + sb * 16384 + h * G::kHalfBytes + ck * 1024 + lane * 16),
                (__attribute__((address_space(3))) void *)(dst + t * G::kHalfBytes + ck * 1024), 16, 0, 0);
        }
        // (every wavefront copies the 512 bytes of one tile's sums, with all 64 lanes - the upper half lands behind them, unused -
        // and several wavefronts may copy the same tile's: no branch around a load into LDS, behind which the compiler would wait
        // for every load in flight in front of the next LDS read)
        if (h == 1)
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void *)(img0 + (wave % NT) * tile_stride + kXFBytes + sb * 512 + (lane & 31) * 16),
                (__attribute__((address_space(3))) void *)(lds + L::kRingBytes + (wave % NT) * 1024), 16, 0, 0);
    };
    // (no fence: the loads that must have landed are waited for by count, and LDS reads have been consumed before a wavefront arrives)
    auto meet = [&](bool all) __attribute__((always_inline)) {
        // (the builtin, not written-out text: the compiler keeps its own count of loads into LDS and would otherwise wait for
        // all of them in front of the first LDS read it cannot tell apart from their destinations)
        if (all) __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        else __builtin_amdgcn_s_waitcnt(0x0F75);       // vmcnt(5)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    f16v acc[NT], p1[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[t][r] = p1[t][r] = 0.f;
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));

    // issue order (two parks): stage(0,0) fetch(0) fetch(1) | per super-block j: stage(j,1) fetch(j+2) | stage(j+1,0);
    // with one park the weight tiles are requested one super-block ahead: stage(0,0) fetch(0) | stage(j,1) fetch(j+1) | stage(j+1,0)
    stage(0, 0);
    asm volatile("" ::: "memory");  // (the counted waits rely on this order of the requests)
    fetch(0);
    asm volatile("" ::: "memory");
    if (L::kParks == 2 && nsb > 1) fetch(1);
    for (int sb = 0; sb < nsb; sb++) {
        // first half: its image (requested one step ago) and this wavefront's weight tile must be there; every wavefront has
        // finished with stage 1, which the second half's image now overwrites
        meet(sb > 0 || nsb == 1 || L::kParks == 1);  // (two parks, super-block 0: only the request of tile 1 may still be out)
        stage(sb, 1);
        const uint8_t *myrow = park0 + (sb % L::kParks) * kParkBytes + col * 144;
        typedef uint32_t Chunk __attribute__((ext_vector_type(4)));
        Chunk rhd = *reinterpret_cast<const Chunk *>(myrow), rc[4];
#pragma unroll
        for (int st = 0; st < 4; st++) rc[st] = *reinterpret_cast<const Chunk *>(myrow + 16 + 32 * st + 16 * kg);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(rhd), "+v"(rc[0]), "+v"(rc[1]), "+v"(rc[2]), "+v"(rc[3])::"memory");
        RawSB cur;
        cur.hd = make_uint4(rhd.x, rhd.y, rhd.z, rhd.w);
#pragma unroll
        for (int st = 0; st < 4; st++) cur.c[st] = make_uint4(rc[st].x, rc[st].y, rc[st].z, rc[st].w);
        __builtin_amdgcn_wave_barrier();
        const bool more = sb + L::kParks < nsb;
        if (more) fetch(sb + L::kParks);
        q4k_tiles_half<NT, 0>(cur, lds, kg, col, magic, p1);
        // second half: the image requested above must be there (the request of a weight tile, issued after it, may still be out)
        meet(!more);
        if (sb + 1 < nsb) stage(sb + 1, 0);
        q4k_tiles_half<NT, 1>(cur, lds + L::kStageBytes, kg, col, magic, p1);
        q4k_tiles_finish<NT>(cur, lds + L::kRingBytes, kg, col, magic, p1, acc);
    }

    if (n < N) {
        // lane holds y[m = 32 t + 8 (r / 4) + 4 kg + r % 4][n] for its K-slice
#pragma unroll
        for (int t = 0; t < NT; t++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + 32 * t + 8 * (r >> 2) + 4 * kg + (r & 3);
                if (m < M) partial[((int64_t)slice * M + m) * set.ntot + set.n0[prob] + n] = acc[t][r];
            }
        }
    }
}

// ---- the activation pre-pass folded into the main kernel --------------------------------------------------------
//
// mmq_q4k_kernel needs two helper launches around it; each costs about four microseconds of which almost nothing is work.
// mmq_q4k_coop_kernel does without the first: the workgroups of a K-slice stage the slice's activations together.
// The unit is one super-block of the image (32 columns x 256 values: 16 KiB of fragments, the sub-block sums and, new,
// one power-of-two scale per column OF THAT SUPER-BLOCK, so that a unit depends on nothing outside itself): a record
// of kRecBytes, kRecStride apart in memory (whole 128-byte lines: a record is written by exactly one workgroup).
//   * Every workgroup converts ONE super-block straight into its LDS: the one it contracts first, j0 = blockIdx.x % nsb.
//     The workgroups blockIdx.x < nsb also publish theirs: record -> memory with write-through stores, then, once
//     those stores are acknowledged, a flag word (agent-scope atomic).
//   * While half of the wavefronts contract super-block j0, the other half (which would otherwise have nothing to
//     do until its first tile) waits for the flags of the slice's other super-blocks and copies their records global ->
//     LDS.  One workgroup barrier later the whole image is in LDS and the loop runs as in mmq_q4k_kernel.
// The flags are never waited for with the data path behind them in doubt: a reader has not touched a record's lines
// before it sees the flag (caches are invalidated where a kernel starts), and the writer's lines have reached memory.
// Nothing here needs the workgroups to be resident together: publishers wait for nobody, and workgroups are dispatched
// in blockIdx order, so a waiting workgroup's publishers are running or done.  Should a flag not appear within
// `spin_ticks` (100 MHz ticks) all the same, the workgroup converts the missing super-blocks itself (same bits).
// The reduction launch that follows clears the flags (mmq_reduce_kernel), so replays of a recorded graph work.
constexpr int kRecTail = kMT * 16 + kMT * 4;       // 640: sub-block sums (16 B per column), inverse scales (fp32 per column)
constexpr int kRecBytes = 16384 + kRecTail;        // 17024
constexpr int kRecStride = 17408;                  // 136 lines of 128 bytes
constexpr int kFlagsPerSlice = 8;
template <int RT> struct Q4KCoopTile {
    static_assert(RT == 4, "LDS budget below is for four row tiles");
    static constexpr int kWaves = RT * kParts, kRows = 32 * RT;
    static constexpr int kMaxSliceSB = 7;
    static constexpr int kLds = kMaxSliceSB * kRecBytes + kWaves * kParkBytes;
    static_assert(kLds <= 160 * 1024, "image + parked tiles exceed LDS");
};

__device__ __forceinline__ float half_wave_max(float v) {  // over the 32 lanes of a wavefront's half
#define GQ_DPP_MAX(ctrl) v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, true)))
    GQ_DPP_MAX(0xB1);   // quad_perm [1,0,3,2]
    GQ_DPP_MAX(0x4E);   // quad_perm [2,3,0,1]
    GQ_DPP_MAX(0x141);  // row_half_mirror
    GQ_DPP_MAX(0x140);  // row_mirror
#undef GQ_DPP_MAX
    return fmaxf(v, __shfl_xor(v, 16, 64));
}

// Super-block `sb` of x (columns m0 .. m0 + 31, values 256 sb .. 256 sb + 255) as one image record in LDS: fragments at
// `frag` (32 slots x 32 columns x 16 bytes, slot and octet order as in stage_x), sums and inverse scales at `tail`.
// All 512 threads: thread = (octet tid % 32, columns tid / 32 and tid / 32 + 16); a column's 32 octets sit in one half
// of a wavefront, so its largest magnitude needs no barrier.
template <bool BF16X>
__device__ __forceinline__ void convert_sb(const void *__restrict__ X, int M, int K, int m0, int sb, uint8_t *frag, uint8_t *tail, int tid) {
    const int oct = tid & 31;
    const int gp = oct >> 3, w8 = oct & 7, high = w8 >> 2, idx8 = w8 & 3;
    const int q = high * 2 + (idx8 & 1), c = 2 * gp + (idx8 >> 1);
    const int slot = c * 4 + q, swz = slot & 15;  // (a super-block is 32 slots: the slice-wide slot index has the same low bits)
    const int j = 2 * gp + high;
    const int jpos = (j & 4) | ((j & 1) << 1) | ((j >> 1) & 1);
    const int64_t k = (int64_t)sb * 256 + 8 * oct;
    float4 lo[2], hi[2];
#pragma unroll
    for (int r = 0; r < 2; r++) load_x8<BF16X>(X, (int64_t)min(m0 + (tid >> 5) + 16 * r, M - 1) * K + k, lo[r], hi[r]);
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const int m = (tid >> 5) + 16 * r;
        const bool ok = m0 + m < M;
        float sc, inv;
        pow2_scale(half_wave_max(ok ? amax8(lo[r], hi[r]) : 0.f), sc, inv);
        if (oct == 0) reinterpret_cast<float *>(tail + kMT * 16)[m] = inv;
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        float4 a = ok ? lo[r] : z, b = ok ? hi[r] : z;
        a.x *= sc; a.y *= sc; a.z *= sc; a.w *= sc; b.x *= sc; b.y *= sc; b.z *= sc; b.w *= sc;
        uint4 o;  // bytes (0,2,1,3,4,6,5,7)
        o.x = pack_h2(a.x, a.z);
        o.y = pack_h2(a.y, a.w);
        o.z = pack_h2(b.x, b.z);
        o.w = pack_h2(b.y, b.w);
        *reinterpret_cast<uint4 *>(frag + slot * (kMT * 16) + (m ^ swz) * 16) = o;
        float sum = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w));
        sum = dpp_quad_sum(sum);  // the four octets of one 32-value sub-block sit in one quad
        if (idx8 == 0) *reinterpret_cast<_Float16 *>(tail + m * 16 + jpos * 2) = (_Float16)sum;
    }
}

template <int RT, bool BF16X>
__global__ __launch_bounds__(64 * RT * kParts) void mmq_q4k_coop_kernel(const void *__restrict__ X, uint8_t *ximg, uint32_t *flags, Q4KSet set,
                                                                        float *__restrict__ partial0, int M, int K, int64_t row_bytes, int m0,
                                                                        int slice_sb, const uint8_t *__restrict__ W2, float *__restrict__ partial2,
                                                                        int spin_ticks) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    __shared__ uint32_t ctl[2];  // [0] wavefronts that have written their part of the published record, [1] super-blocks that did not arrive
    int prob = 0;
#pragma unroll
    for (int j = 1; j < kMaxSet; j++)
        if (j < set.count && (int)blockIdx.x >= set.wg0[j]) prob = j;
    const uint8_t *__restrict__ W = blockIdx.z ? W2 : set.W[prob];
    float *__restrict__ partial = blockIdx.z ? partial2 : partial0;
    const int N = set.N[prob], xblk = (int)blockIdx.x - set.wg0[prob];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 5, col = lane & 31;
    const int rt = wave % RT, par = wave / RT;
    const int slice = blockIdx.y, nslices = gridDim.y;
    const int nsb = ((K >> 8) - slice + nslices - 1) / nslices;  // slice s holds super-blocks s, s + nslices, ... of every row
    const int n = xblk * (32 * RT) + rt * 32 + col;
    const int mt = m0 / kMT;
    uint8_t *img = ximg + ((size_t)mt * nslices + slice) * ((size_t)Q4KCoopTile<RT>::kMaxSliceSB * kRecStride);
    uint32_t *flg = flags + ((size_t)mt * nslices + slice) * kFlagsPerSlice;
    // the super-block this workgroup stages itself and contracts first; position p of its sequence is super-block (j0 + p) % nsb
    const int j0 = (int)blockIdx.x % nsb;
    const bool publisher = blockIdx.z == 0 && (int)blockIdx.x < nsb;
    auto sb_at = [&](int p) { const int sbl = j0 + p; return sbl >= nsb ? sbl - nsb : sbl; };

    const int xs_off = slice_sb * 16384;  // tails follow the fragments
    const int row0 = xblk * (32 * RT) + rt * 32;
    const uint8_t *wtile = W + (int64_t)min(row0, N - 1) * row_bytes + slice * 144;
    uint32_t csrc[kParkLoads];  // (byte offsets from the first row of the tile: mmq_supported keeps 31 rows below 2^32 bytes)
#pragma unroll
    for (int l = 0; l < kParkLoads; l++) {
        const int c = min(lane + 64 * l, 32 * 9 - 1);
        csrc[l] = (uint32_t)(min(row0 + c / 9, N - 1) - min(row0, N - 1)) * (uint32_t)row_bytes + (uint32_t)((c % 9) * 16);
    }
    uint8_t *park = lds + xs_off + slice_sb * kRecTail + wave * kParkBytes;
    auto fetch = [&](int sbl) __attribute__((always_inline)) {
        const uint8_t *base = wtile + sbl * nslices * 144;
#pragma unroll
        for (int l = 0; l < kParkLoads; l++)
            if (64 * l + 64 <= 32 * 9 || lane < 32 * 9 - 64 * l)  // (the last instruction carries 32 chunks)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(base + csrc[l]),
                                                 (__attribute__((address_space(3))) void *)(park + l * 1024), 16, 0, 0);
    };
    if (par < nsb) fetch(sb_at(par));  // the weights of the first tile travel while the activations are staged
    const uint8_t *myrow = park + col * 144;
    if (tid == 0) { ctl[0] = 0u; ctl[1] = 0u; }
    convert_sb<BF16X>(X, M, K, m0, slice + j0 * nslices, lds + j0 * 16384, lds + xs_off + j0 * kRecTail, tid);
    __syncthreads();  // this workgroup's own super-block is staged

    f16v acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));
    // position p: wait for the parked tile, pick out this lane's part, request the tile two positions on, contract
    auto contract_at = [&](int p) __attribute__((always_inline)) {
        const int sbl = sb_at(p);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        typedef uint32_t Chunk __attribute__((ext_vector_type(4)));
        Chunk rhd = *reinterpret_cast<const Chunk *>(myrow), rc[4];
#pragma unroll
        for (int st = 0; st < 4; st++) rc[st] = *reinterpret_cast<const Chunk *>(myrow + 16 + 32 * st + 16 * kg);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(rhd), "+v"(rc[0]), "+v"(rc[1]), "+v"(rc[2]), "+v"(rc[3])::"memory");
        RawSB cur;
        cur.hd = make_uint4(rhd.x, rhd.y, rhd.z, rhd.w);
#pragma unroll
        for (int st = 0; st < 4; st++) cur.c[st] = make_uint4(rc[st].x, rc[st].y, rc[st].z, rc[st].w);
        __builtin_amdgcn_wave_barrier();
        if (p + kParts < nsb) fetch(sb_at(p + kParts));
        const uint8_t *tail = lds + xs_off + sbl * kRecTail;
        q4k_contract_sb<true>(cur, lds, tail, reinterpret_cast<const float *>(tail + kMT * 16), sbl, kg, col, magic, acc);
    };

    if (par == 0) {
        contract_at(0);
    } else {
        if (publisher) {  // the record of super-block j0 goes to memory, a quarter per wavefront
            for (int c = rt * 64 + lane; c < kRecBytes / 16; c += RT * 64) {
                const uint8_t *src = c < 1024 ? lds + j0 * 16384 + c * 16 : lds + xs_off + j0 * kRecTail + (c - 1024) * 16;
                store_through(img + (size_t)j0 * kRecStride + (size_t)c * 16, *reinterpret_cast<const uint4 *>(src));
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores have been acknowledged
            if (lane == 0 && atomicAdd(&ctl[0], 1u) == (uint32_t)(RT - 1))  // the last of the four wavefronts raises the flag
                __hip_atomic_store(flg + j0, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // the slice's other super-blocks: wait until they are published (bounded), then copy them in
        const uint32_t want = (1u << nsb) - 1u;
        uint32_t have;
        {
            const unsigned long long t0 = wall_clock64();
            for (;;) {
                uint32_t v = 1u;
                if (lane < nsb && lane != j0) v = __hip_atomic_load(flg + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                have = (uint32_t)__ballot(v != 0u) & want;
                if (have == want || wall_clock64() - t0 >= (unsigned long long)spin_ticks) break;
                __builtin_amdgcn_s_sleep(1);
            }
        }
        if (have != want && lane == 0) atomicOr(&ctl[1], want & ~have);
        asm volatile("" ::: "memory");
        for (int sbl = 0; sbl < nsb; sbl++) {
            if (sbl == j0 || !((have >> sbl) & 1u)) continue;
            const uint8_t *rec = img + (size_t)sbl * kRecStride;
#pragma unroll
            for (int i = 0; i < 16 / RT; i++) {  // fragments: 16 KiB, 1 KiB per instruction
                const int kib = rt + RT * i;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(rec + kib * 1024 + lane * 16),
                                                 (__attribute__((address_space(3))) void *)(lds + sbl * 16384 + kib * 1024), 16, 0, 0);
            }
            if (rt == 0 && lane < kRecTail / 16)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(rec + 16384 + lane * 16),
                                                 (__attribute__((address_space(3))) void *)(lds + xs_off + sbl * kRecTail), 16, 0, 0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (a barrier does not wait for loads in flight)
    }
    __syncthreads();  // the image is complete
    if (const uint32_t missing = ctl[1]) {  // (only after a wait ran out) the workgroup stages what did not arrive itself
        for (int sbl = 0; sbl < nsb; sbl++)
            if ((missing >> sbl) & 1u) convert_sb<BF16X>(X, M, K, m0, slice + sbl * nslices, lds + sbl * 16384, lds + xs_off + sbl * kRecTail, tid);
        __syncthreads();
    }
    for (int p = par == 0 ? kParts : par; p < nsb; p += kParts) contract_at(p);

    // wavefronts 1..kParts-1 of a row tile hand their 32 x 32 partial tiles to wavefront 0 through LDS
    __syncthreads();
    float *xch = reinterpret_cast<float *>(lds) + rt * ((kParts - 1) * 16 * 64);
    if (par > 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) xch[((par - 1) * 16 + r) * 64 + lane] = acc[r];
    }
    __syncthreads();
    if (par == 0 && n < N) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = m0 + 8 * (r >> 2) + 4 * kg + (r & 3);
            float v = acc[r];
#pragma unroll
            for (int p = 0; p < kParts - 1; p++) v += xch[(p * 16 + r) * 64 + lane];
            if (m < M) partial[((int64_t)slice * M + m) * set.ntot + set.n0[prob] + n] = v;
        }
    }
}

// y[m][n] = act(sum_s partial[s][m][n] + bias[n]); N % 4 == 0 is guaranteed by the caller.  With a second
// set of partial sums (the other matrix of a gated pair) the result is multiplied by
// sum_s partial2[s][m][n] + bias2[n]; a residual (which may be Y itself) is added last.
// xscale[slice][M]: factor of each slice's partial sums of row m (the activations of a slice were scaled by its inverse).
__global__ __launch_bounds__(256) void mmq_reduce_kernel(const float *__restrict__ partial, const float *__restrict__ partial2, int nslices,
                                                         int64_t MN, int N, const float *__restrict__ bias, const float *__restrict__ bias2,
                                                         int act, const float *residual, float *Y, const float *__restrict__ xscale,
                                                         const float *__restrict__ xss, float eps, float inv_k, uint32_t *flags, int nflags) {
    // (the main kernel that stages the activations itself raised these flags; the stream orders this kernel behind it)
    if (blockIdx.x == 0)
        for (int f = threadIdx.x; f < nflags; f += blockDim.x) flags[f] = 0u;
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= MN) return;
    const bool small = MN <= (int64_t)INT32_MAX;  // (32-bit divisions are a fraction of the cost of 64-bit ones)
    const int M = small ? (int)((uint32_t)MN / (uint32_t)N) : (int)(MN / N);
    const int m = small ? (int)((uint32_t)i / (uint32_t)N) : (int)(i / N);
    // Slices are added in order, eight at a time: their loads (each a trip to another XCD's freshly written
    // lines) are all issued before the first sum needs one; a slice past the end re-reads the last and is not added.
    // xss: the activations carry an RMS normalisation whose 1 / sqrt(mean(x^2) + eps) is applied here, to the finished sums.
    auto total = [&](const float *p, const float *b) {
        float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
        float ss = 0.f;
        for (int k0 = 0; k0 < nslices; k0 += 8) {
            float4 v[8];
            float f[8], q[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int k = min(k0 + j, nslices - 1);
                v[j] = *reinterpret_cast<const float4 *>(p + (int64_t)k * MN + i);
                f[j] = xscale ? xscale[(int64_t)k * M + m] : 1.f;  // (no slice scales: the main kernel has applied its own)
                q[j] = xss ? xss[(int64_t)k * M + m] : 0.f;
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const bool in = k0 + j < nslices;
                s.x = in ? fmaf(v[j].x, f[j], s.x) : s.x; s.y = in ? fmaf(v[j].y, f[j], s.y) : s.y;
                s.z = in ? fmaf(v[j].z, f[j], s.z) : s.z; s.w = in ? fmaf(v[j].w, f[j], s.w) : s.w;
                ss = in ? ss + q[j] : ss;
            }
        }
        if (xss) {
            const float r = sqrtf(ss * inv_k + eps);
            s.x /= r; s.y /= r; s.z /= r; s.w /= r;
        }
        if (b) {
            const float4 v = *reinterpret_cast<const float4 *>(b + (int)(i % N));
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        return s;
    };
    const float4 s = total(partial, bias);
    float4 v = make_float4(apply_act(act, s.x), apply_act(act, s.y), apply_act(act, s.z), apply_act(act, s.w));
    if (partial2) {
        const float4 u = total(partial2, bias2);
        v.x *= u.x; v.y *= u.y; v.z *= u.z; v.w *= u.w;
    }
    if (residual) {
        const float4 r = *reinterpret_cast<const float4 *>(residual + i);
        v.x += r.x; v.y += r.y; v.z += r.z; v.w += r.w;
    }
    *reinterpret_cast<float4 *>(Y + i) = v;
}

// [xscale: nslices x M][xss: nslices x M] (the second only used with a normalisation)
size_t mmq_scale_bytes(int nslices, int64_t M) { return ((size_t)2 * nslices * M * sizeof(float) + 255) & ~(size_t)255; }
float *mmq_xss(const float *xscale, int nslices, int64_t M) { return const_cast<float *>(xscale) + (size_t)nslices * M; }

int launch_mmq_reduce(const float *partial, const float *partial2, const float *xscale, int nslices, int64_t M, int64_t K, int64_t N,
                      const float *bias, int act, float *y, const MmqExtra *ex, hipStream_t s, uint32_t *flags = nullptr, int nflags = 0) {
    const int64_t MN = M * N;
    const RmsNorm *norm = ex ? ex->norm : nullptr;
    // (workgroups of 64 threads while 256 would leave CUs without one: the kernel is one round trip to memory long)
    const int threads = MN / 4 / 256 >= 2 * device_cu_count() ? 256 : 64;
    return launch(mmq_reduce_kernel, dim3((unsigned)((MN / 4 + threads - 1) / threads)), dim3(threads), 0, s, partial, partial2, nslices, MN, (int)N, bias,
                  ex ? ex->bias2 : nullptr, act, ex ? ex->residual : nullptr, y, xscale, norm ? mmq_xss(xscale, nslices, M) : nullptr,
                  norm ? norm->eps : 0.f, 1.0f / (float)K, flags, nflags);
}


// The reduction for a set of matrices contracted in one launch: partial[slice][m][ntot] holds their columns side by
// side; matrix p's columns n0[p] .. go to its own y[p] ([M, N[p]]) with its own bias and activation.  Every N[p] % 4 == 0.
struct MmqSetOut {
    const float *bias[kMaxSet];
    float *y[kMaxSet];
    int N[kMaxSet], n0[kMaxSet], act[kMaxSet];
    int count, ntot;
};
__global__ __launch_bounds__(256) void mmq_reduce_set_kernel(const float *__restrict__ partial, int nslices, int M, MmqSetOut out,
                                                             const float *__restrict__ xscale, const float *__restrict__ xss, float eps,
                                                             float inv_k, uint32_t *flags, int nflags) {
    if (blockIdx.x == 0)
        for (int f = threadIdx.x; f < nflags; f += blockDim.x) flags[f] = 0u;
    const int64_t total = (int64_t)M * out.ntot;
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= total) return;
    const int m = (int)(i / out.ntot), nt = (int)(i - (int64_t)m * out.ntot);
    int p = 0;
#pragma unroll
    for (int j = 1; j < kMaxSet; j++)
        if (j < out.count && nt >= out.n0[j]) p = j;
    const int n = nt - out.n0[p];
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    float ss = 0.f;
    for (int k0 = 0; k0 < nslices; k0 += 8) {  // (all of a round's loads are issued before the first sum needs one)
        float4 v[8];
        float f[8], q[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int k = min(k0 + j, nslices - 1);
            v[j] = *reinterpret_cast<const float4 *>(partial + (int64_t)k * total + i);
            f[j] = xscale ? xscale[(int64_t)k * M + m] : 1.f;
            q[j] = xss ? xss[(int64_t)k * M + m] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const bool in = k0 + j < nslices;
            s.x = in ? fmaf(v[j].x, f[j], s.x) : s.x; s.y = in ? fmaf(v[j].y, f[j], s.y) : s.y;
            s.z = in ? fmaf(v[j].z, f[j], s.z) : s.z; s.w = in ? fmaf(v[j].w, f[j], s.w) : s.w;
            ss = in ? ss + q[j] : ss;
        }
    }
    if (xss) {
        const float r = sqrtf(ss * inv_k + eps);
        s.x /= r; s.y /= r; s.z /= r; s.w /= r;
    }
    if (out.bias[p]) {
        const float4 b = *reinterpret_cast<const float4 *>(out.bias[p] + n);
        s.x += b.x; s.y += b.y; s.z += b.z; s.w += b.w;
    }
    const int act = out.act[p];
    *reinterpret_cast<float4 *>(out.y[p] + (int64_t)m * out.N[p] + n) =
        make_float4(apply_act(act, s.x), apply_act(act, s.y), apply_act(act, s.z), apply_act(act, s.w));
}

// ---- small batches of the 32-value-block formats (Q8_0, Q4_0, IQ4_NL) --------------------------------------
//
// Same plan as the Q4_K kernel above, simpler arithmetic: K is split in slices of S = 512 or 1024
// values (the smaller count of slices that still gives the chip a few hundred workgroups); a
// workgroup keeps the slice of x for 32 batch columns in LDS as fp16 octets in natural order
// ([octet][column][8 values], copied global -> LDS from an image a pre-pass wrote) and streams
// 128 rows of W past it: 8 wavefronts = 4 row tiles of 32 x 2 interleaved sequences of 256-value
// stretches (8 blocks).
//
// Loading: a load instruction whose 64 lanes touch 64 different cache lines (one W row per lane)
// occupies the texture addresser for ~2.4 cycles per lane, which alone holds a kernel at
// ~1.5 TB/s.  So a wavefront reads a stretch of its 32 rows as 16-byte chunks in row-major chunk
// order (consecutive lanes = consecutive chunks of one row: 17 per row for Q8_0, 9 for Q4_0),
// parks them in a private piece of LDS and only then lets lane (col = lane % 32, kg = lane / 32)
// pick out the codes of W row `col`:
//   Q8_0: bytes 16 kg .. 16 kg + 15 of block b -> octets 4 b + 2 kg + j, j = 0, 1;
//   Q4_0: bytes 8 kg .. 8 kg + 7: low nibbles -> octet 4 b + kg, high nibbles -> octet 4 b + 2 + kg.
// Blocks start 2 bytes off a dword boundary every other block; the LDS reads are dword windows
// plus a funnel shift (which block is odd is known at compile time).
// Codes become exact fp16 integers (magic number 1024 + code, one packed add), two MFMAs contract
// a block against the activations, and the block's partial tile is scaled by d in fp32:
// x -> fp16 is the only rounding that is not fp32.
template <int T> struct B32;
template <> struct B32<kQ8_0> {
    static constexpr int kBlockBytes = 34, kWin = 5;  // dwords that cover a lane's 16 codes from the dword at or below them
    static __device__ __forceinline__ int code_byte(int kg) { return 2 + 16 * kg; }
    static __device__ __forceinline__ int octet(int b, int kg, int j) { return 4 * b + 2 * kg + j; }
    // fragment j: values 8 j .. 8 j + 7 of the lane's sixteen, as fp16 pairs (0,2) (1,3) (4,6) (5,7);
    // c[0..3] are the four code dwords
    static __device__ __forceinline__ h8 frag(const uint32_t *c, int j, uint32_t magic) {
        const uint32_t a = c[2 * j] ^ 0x80808080u, b = c[2 * j + 1] ^ 0x80808080u;  // code + 128, unsigned
        const h2 off = as_h2(0xE480E480u);  // (-1152, -1152) = -(1024 + 128)
        uint4 o;
        o.x = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, a, 0x07020700u)) + off);  // bytes (a0, 0x64, a2, 0x64)
        o.y = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, a, 0x07030701u)) + off);
        o.z = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, b, 0x07020700u)) + off);
        o.w = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, b, 0x07030701u)) + off);
        return __builtin_bit_cast(h8, o);
    }
};
template <> struct B32<kQ4_0> {
    static constexpr int kBlockBytes = 18, kWin = 3;
    static __device__ __forceinline__ int code_byte(int kg) { return 2 + 8 * kg; }
    static __device__ __forceinline__ int octet(int b, int kg, int j) { return 4 * b + 2 * j + kg; }
    // fragment 0: low nibbles, fragment 1: high nibbles of the lane's eight bytes (c[0..1]), minus 8
    static __device__ __forceinline__ h8 frag(const uint32_t *c, int j, uint32_t magic) {
        const uint32_t a = c[0] >> (4 * j), b = c[1] >> (4 * j);
        const h2 off = as_h2(0xE408E408u);  // (-1032, -1032) = -(1024 + 8)
        uint4 o;
        o.x = __builtin_bit_cast(uint32_t, magic_pair(a, 0x000F000Fu, magic) + off);       // nibbles of bytes (0, 2)
        o.y = __builtin_bit_cast(uint32_t, magic_pair(a >> 8, 0x000F000Fu, magic) + off);  // (1, 3)
        o.z = __builtin_bit_cast(uint32_t, magic_pair(b, 0x000F000Fu, magic) + off);
        o.w = __builtin_bit_cast(uint32_t, magic_pair(b >> 8, 0x000F000Fu, magic) + off);
        return __builtin_bit_cast(h8, o);
    }
};

// IQ4_NL: the layout of Q4_0 with a 16-entry code book instead of nibble - 8.
template <> struct B32<kIQ4_NL> {
    static constexpr int kBlockBytes = 18, kWin = 3;
    static __device__ __forceinline__ int code_byte(int kg) { return 2 + 8 * kg; }
    static __device__ __forceinline__ int octet(int b, int kg, int j) { return 4 * b + 2 * j + kg; }
    // four code-book entries (int8, as bytes) for the four nibble indices in the bytes of idx
    static __device__ __forceinline__ uint32_t book(uint32_t idx) {
        const uint32_t t0 = 0xBFAD9881u, t1 = 0xF6EADDCFu, t2 = 0x26190D01u, t3 = 0x71594535u;  // -127 .. 113, four per dword
        const uint32_t low3 = idx & 0x07070707u;
        const uint32_t lo = __builtin_amdgcn_perm(t1, t0, low3), hi = __builtin_amdgcn_perm(t3, t2, low3);
        return __builtin_amdgcn_perm(hi, lo, 0x03020100u | ((idx & 0x08080808u) >> 1));  // byte i from hi when bit 3 of index i is set
    }
    static __device__ __forceinline__ h8 frag(const uint32_t *c, int j, uint32_t magic) {
        const uint32_t a = book((c[0] >> (4 * j)) & 0x0F0F0F0Fu) ^ 0x80808080u;  // entry + 128, unsigned
        const uint32_t b = book((c[1] >> (4 * j)) & 0x0F0F0F0Fu) ^ 0x80808080u;
        const h2 off = as_h2(0xE480E480u);  // (-1152, -1152) = -(1024 + 128)
        uint4 o;
        o.x = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, a, 0x07020700u)) + off);
        o.y = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, a, 0x07030701u)) + off);
        o.z = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, b, 0x07020700u)) + off);
        o.w = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, b, 0x07030701u)) + off);
        return __builtin_bit_cast(h8, o);
    }
};

constexpr int kB32Stretch = 8;    // blocks per stretch (256 values)

template <int T> struct B32Geom {
    static constexpr int kStretchBytes = kB32Stretch * B32<T>::kBlockBytes;  // 272 / 144 per row
    static constexpr int kCPR = kStretchBytes / 16;                          // 16-byte chunks per row: 17 / 9
    static constexpr int kChunks = 32 * kCPR;                                // per wavefront and stretch
    static constexpr int kLoads = (kChunks + 63) / 64;                       // 9 / 5 load instructions
    static constexpr int kWaveLds = 32 * kStretchBytes + 16;                 // + slack: a window may end past the last row
};

// Image of x for the main kernel: [column tile][slice][octet of the slice][32 columns][8 fp16 in the
// order (0,2,1,3,4,6,5,7)]; columns beyond M and values beyond K are zero.  One workgroup converts 8
// columns of one slice (S / 256 octets per thread, consecutive threads on consecutive octets of a
// column) and scales each column's slice by a power of two (pow2_scale); xscale[slice][M] receives the
// inverse factors.  grid = column tiles x slices x 4.
template <bool BF16X>
__global__ __launch_bounds__(256) void mmq_b32_xprep_kernel(const void *__restrict__ X, uint8_t *__restrict__ ximg, float *__restrict__ xscale,
                                                            int M, int K, int S, int nslices, const float *__restrict__ gain, float gain_offset,
                                                            float *__restrict__ xss) {
    __shared__ uint32_t red[8];
    __shared__ float red_ss[8][2];  // a column's slice is one or two wavefronts' worth of octets
    const int tid = threadIdx.x;
    const int rg = (int)blockIdx.x & 3, ts = (int)blockIdx.x >> 2;
    const int slice = ts % nslices, mt = ts / nslices;
    const int opers = S / 8, its = S / 256;  // octets per column and slice; items per thread
    if (tid < 8) {
        red[tid] = 0u;
        red_ss[tid][0] = 0.f;
        red_ss[tid][1] = 0.f;
    }
    __syncthreads();
    float4 a[4], b[4];
#pragma unroll
    for (int it = 0; it < 4; it++) {
        a[it] = make_float4(0.f, 0.f, 0.f, 0.f);
        b[it] = a[it];
        if (it < its) {
            const int j = it * 256 + tid, c = j / opers, oct = j - c * opers;
            const int k = slice * S + oct * 8, row = mt * kMT + rg * 8 + c;
            const bool ok = row < M && k < K;  // K % 32 == 0: an octet is inside or outside as a whole
            if (ok) load_x8<BF16X>(X, (int64_t)row * K + k, a[it], b[it]);
            if (xss) {
                const float ss = wave_sum(sumsq8(a[it], b[it]));
                if ((tid & 63) == 0) red_ss[c][(oct >> 6) & 1] = ss;
                if (gain && ok) apply_gain8(gain, gain_offset, k, a[it], b[it]);
            }
            const float am = wave_max(amax8(a[it], b[it]));  // a wavefront's 64 octets belong to one column
            if ((tid & 63) == 0) atomicMax(&red[c], __builtin_bit_cast(uint32_t, am));  // (non-negative floats order like their bits)
        }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; it++) {
        if (it < its) {
            const int j = it * 256 + tid, c = j / opers, oct = j - c * opers;
            const int m = rg * 8 + c, row = mt * kMT + m;
            float sc, inv;
            pow2_scale(__builtin_bit_cast(float, red[c]), sc, inv);
            if (oct == 0 && row < M) {
                xscale[(size_t)slice * M + row] = inv;
                if (xss) xss[(size_t)slice * M + row] = red_ss[c][0] + red_ss[c][1];
            }
            const float4 p = a[it], q = b[it];
            const size_t g = (((size_t)mt * nslices + slice) * opers + oct) * 32 + m;
            reinterpret_cast<uint4 *>(ximg)[g] = make_uint4(pack_h2(p.x * sc, p.z * sc), pack_h2(p.y * sc, p.w * sc), pack_h2(q.x * sc, q.z * sc),
                                                            pack_h2(q.y * sc, q.w * sc));
        }
    }
}

// partial[slice][m][n] = sum over the slice's k of x[m][k] * w[n][k];  grid (row ranges, slices, column tiles)
// RT row tiles of 32 W rows per workgroup, two wavefronts each.  K % 256 == 0.
// LDS: [activation image: S * 64 bytes][per wavefront: one stretch of 32 rows]
template <int T, int RT>
__global__ __launch_bounds__(RT * 128) void mmq_b32_kernel(const uint8_t *__restrict__ ximg, const uint8_t *__restrict__ W0,
                                                           float *__restrict__ partial0, int M, int K, int N, int64_t row_bytes, int S, int mtiles,
                                                           const uint8_t *__restrict__ W2, float *__restrict__ partial2) {
    // blockIdx.z >= mtiles: the second matrix of a gated pair (same activation image, its own partial sums)
    const bool second = (int)blockIdx.z >= mtiles;
    const uint8_t *__restrict__ W = second ? W2 : W0;
    float *__restrict__ partial = second ? partial2 : partial0;
    typedef B32<T> F;
    typedef B32Geom<T> G;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 5, col = lane & 31;
    const int rt = wave % RT, par = wave / RT;
    const int slice = blockIdx.y, nslices = gridDim.y, mt = second ? (int)blockIdx.z - mtiles : (int)blockIdx.z;
    const int img_bytes = S * 64;
    const int kstretches = K >> 8, t0 = slice * (S >> 8);      // stretches of a row; first stretch of the slice
    const int n0 = (blockIdx.x * RT + rt) * 32;                // first W row of this wavefront's tile
    uint8_t *park = lds + img_bytes + wave * G::kWaveLds;      // this wavefront's stretch

    // the slice's activation image goes straight from global memory into LDS (no registers)
    {
        const uint8_t *img = ximg + ((size_t)mt * nslices + slice) * img_bytes;
        for (int i = wave; i < img_bytes / 1024; i += 2 * RT)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(img + i * 1024 + lane * 16),
                                             (__attribute__((address_space(3))) void *)(lds + i * 1024), 16, 0, 0);
    }
    // Wavefront `par` takes stretches par, par + 2, ... of the slice; stretches beyond K re-read the
    // row's last one (their activations are zero in the image).  Chunk c = lane + 64 i of a stretch is
    // chunk c % kCPR of row c / kCPR.
    uint32_t coff[G::kLoads];  // byte offset of this lane's chunks from the stretch's start in row n0
#pragma unroll
    for (int i = 0; i < G::kLoads; i++) {
        const int c = min(lane + 64 * i, G::kChunks - 1);
        coff[i] = (uint32_t)min(c / G::kCPR, max(N - 1 - n0, 0)) * (uint32_t)row_bytes + (uint32_t)(c % G::kCPR) * 16u;
    }
    const uint8_t *wtile = W + (int64_t)min(n0, N - 1) * row_bytes;
    typedef uint32_t Chunk __attribute__((ext_vector_type(4)));
    typedef Chunk ChunkA4 __attribute__((aligned(4)));  // rows are only 4-byte aligned in general
    Chunk buf[G::kLoads];
    auto fetch = [&](int i) __attribute__((always_inline)) {  // i-th stretch of this wavefront
        const uint8_t *base = wtile + (int64_t)min(t0 + 2 * i + par, kstretches - 1) * G::kStretchBytes;
#pragma unroll
        for (int l = 0; l < G::kLoads; l++) buf[l] = *reinterpret_cast<const ChunkA4 *>(base + coff[l]);
    };
    fetch(0);
    // a barrier does not wait for loads in flight: every wavefront's share of the image copy must have landed in LDS
    // before it arrives (loads complete in order, so this also waits for the first stretch, which is needed next anyway)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    f16v acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));
    const int ns = S >> 9;  // stretches per wavefront: 1 or 2
    const uint8_t *myrow = park + col * G::kStretchBytes;
    for (int g = 0; g < ns; g++) {
        // park the stretch (LDS operations of one wavefront execute in order; no other wavefront reads it)
#pragma unroll
        for (int l = 0; l < G::kLoads; l++)
            if (lane + 64 * l < G::kChunks) *reinterpret_cast<Chunk *>(park + (lane + 64 * l) * 16) = buf[l];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (g + 1 < ns) fetch(g + 1);
        const int sb = 8 * (2 * g + par);  // first block of the stretch within the slice
#pragma unroll
        for (int j = 0; j < kB32Stretch; j++) {
            const int b = sb + j;
            const h8 x0 = *reinterpret_cast<const h8 *>(lds + (F::octet(b, kg, 0) * kMT + col) * 16);
            const h8 x1 = *reinterpret_cast<const h8 *>(lds + (F::octet(b, kg, 1) * kMT + col) * 16);
            // the lane's codes: a dword window from the dword at or below them, funnel-shifted when
            // the block starts 2 bytes off (every even block: 34 j and 18 j are 2 mod 4 for odd j,
            // and the codes start 2 bytes into the block)
            const int at = j * F::kBlockBytes + F::code_byte(kg);
            const uint32_t *wp = reinterpret_cast<const uint32_t *>(myrow + (at & ~3));
            uint32_t w[F::kWin], c[F::kWin - 1];
#pragma unroll
            for (int q = 0; q < F::kWin; q++) w[q] = wp[q];
#pragma unroll
            for (int q = 0; q < F::kWin - 1; q++) c[q] = (j & 1) ? w[q] : __builtin_amdgcn_alignbit(w[q + 1], w[q], 16);
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(myrow + j * F::kBlockBytes));
            f16v p;
#pragma unroll
            for (int r = 0; r < 16; r++) p[r] = 0.f;
            p = __builtin_amdgcn_mfma_f32_32x32x16_f16(x0, F::frag(c, 0, magic), p, 0, 0, 0);
            p = __builtin_amdgcn_mfma_f32_32x32x16_f16(x1, F::frag(c, 1, magic), p, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] = fmaf(d, p[r], acc[r]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the reads above are done before the next stretch is parked
        __builtin_amdgcn_wave_barrier();
    }

    // the second wavefront of a row tile hands its 32 x 32 partial tile to the first through LDS
    __syncthreads();
    float *xch = reinterpret_cast<float *>(lds) + rt * (16 * 64);
    if (par > 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) xch[r * 64 + lane] = acc[r];
    }
    __syncthreads();
    const int n = n0 + col;
    if (par == 0 && n < N) {
        // lane holds y[m = 8 (r / 4) + 4 kg + r % 4][n] for its K-slice
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = mt * kMT + 8 * (r >> 2) + 4 * kg + (r & 3);
            if (m < M) partial[((int64_t)slice * M + m) * N + n] = acc[r] + xch[r * 64 + lane];
        }
    }
}

// ---- the 18-byte-block formats at more than 32 batch rows -------------------------------------------------------
//
// A 256-value stretch of Q4_0 or IQ4_NL is 144 bytes of a row, like a Q4_K super-block, and rows are 16-byte aligned when K
// is a multiple of 256: mmq_q4k_tiles_kernel's plan carries over as it stands - eight wavefronts with a row tile of 32 rows
// each, weight tiles parked in LDS by DMA two stretches ahead, the images of up to four tiles of 32 batch rows staged half
// a stretch (four blocks) at a time through a ring of two stages with counted waits - and only the arithmetic differs:
// per block two MFMAs per tile against fragments converted ONCE for all tiles, and the block's d applied to each tile's
// sums in fp32.  Slices are S consecutive values (512 or 1024), the image is mmq_b32_xprep_kernel's.
int tiles_together_mode();

template <int NT> struct B32TilesOf {  // LDS: [ring: 2 stages x NT halves of 8 KiB][two parked stretches per wavefront]
    static constexpr int kStageBytes = NT * Q4KTiles::kHalfBytes;
    static constexpr int kRingBytes = 2 * kStageBytes;
    static constexpr int kParks = 2;
    static constexpr int kLds = kRingBytes + kParks * Q4KTiles::kWaves * kParkBytes + 16;  // (+ slack: a code window may end past the last row)
    static_assert(kLds <= 160 * 1024, "images + parked tiles exceed LDS");
};

template <int T, int NT>
__global__ __launch_bounds__(64 * Q4KTiles::kWaves) void mmq_b32_tiles_kernel(const uint8_t *__restrict__ ximg, const uint8_t *__restrict__ W0,
                                                                               float *__restrict__ partial0, int M, int K, int N, int64_t row_bytes, int S,
                                                                               int m0, const uint8_t *__restrict__ W2, float *__restrict__ partial2) {
    typedef B32<T> F;
    typedef Q4KTiles G;
    typedef B32TilesOf<NT> L;
    static_assert(F::kBlockBytes == 18 && kB32Stretch * F::kBlockBytes * 32 == kParkBytes, "a stretch of 32 rows is a parked tile of 32 x 144 bytes");
    static_assert(kParkLoads == 5, "the counted waits below assume five load instructions per weight tile");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint8_t *__restrict__ W = blockIdx.z ? W2 : W0;
    float *__restrict__ partial = blockIdx.z ? partial2 : partial0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 5, col = lane & 31;
    const int slice = blockIdx.y, nslices = gridDim.y;
    const int per_slice = S >> 8, first = slice * per_slice;
    const int nst = min(per_slice, (K >> 8) - first);  // stretches of this slice (at least one)
    const int row0 = (int)blockIdx.x * G::kRows + wave * 32;
    const int n = row0 + col;  // this lane's weight row

    const uint8_t *wtile = W + (int64_t)min(row0, N - 1) * row_bytes + (int64_t)first * 144;
    uint32_t csrc[kParkLoads];
#pragma unroll
    for (int l = 0; l < kParkLoads; l++) {
        const int c = min(lane + 64 * l, 32 * 9 - 1);
        csrc[l] = (uint32_t)(min(row0 + c / 9, N - 1) - min(row0, N - 1)) * (uint32_t)row_bytes + (uint32_t)((c % 9) * 16);
    }
    uint8_t *const park0 = lds + L::kRingBytes + wave * (L::kParks * kParkBytes);
    auto fetch = [&](int j) __attribute__((always_inline)) {  // stretch j of the slice -> park j % 2: exactly kParkLoads load instructions
        const uint8_t *base = wtile + j * 144;
        uint8_t *park = park0 + (j & 1) * kParkBytes;
#pragma unroll
        for (int l = 0; l < kParkLoads; l++)
            if (64 * l + 64 <= 32 * 9 || lane < 32 * 9 - 64 * l)  // (the last instruction carries 32 chunks)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(base + csrc[l]),
                                                 (__attribute__((address_space(3))) void *)(park + l * 1024), 16, 0, 0);
    };
    // tile t's image of this slice: [octet][32 columns][16 bytes], 32 octets (16 KiB) per stretch
    const size_t img_bytes = (size_t)S * 64;
    const uint8_t *img0 = ximg + ((size_t)(m0 / kMT) * nslices + slice) * img_bytes;
    const size_t tile_stride = (size_t)nslices * img_bytes;
    auto stage = [&](int j, int h) __attribute__((always_inline)) {  // half h (four blocks) of stretch j of every tile -> ring stage h
        uint8_t *dst = lds + h * L::kStageBytes;
        for (int i = wave; i < NT * 8; i += G::kWaves) {
            const int t = i >> 3, ck = i & 7;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void *)(img0 + t * tile_stride + j * 16384 + h * G::kHalfBytes + ck * 1024 + lane * 16),
                (__attribute__((address_space(3))) void *)(dst + t * G::kHalfBytes + ck * 1024), 16, 0, 0);
        }
    };
    auto meet = [&](bool all) __attribute__((always_inline)) {  // (see mmq_q4k_tiles_kernel)
        if (all) __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        else __builtin_amdgcn_s_waitcnt(0x0F75);       // vmcnt(5)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    f16v acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[t][r] = 0.f;
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));

    // four blocks of the parked stretch (read in place: the park is not requested again before the stretch is done) against
    // ring stage H: block b's codes are lane (col, kg)'s eight bytes, a dword window from the dword at or below them,
    // funnel-shifted when the block starts 2 bytes off a dword (every even block)
    auto half = [&](auto hc, const uint8_t *myrow) __attribute__((always_inline)) {
        constexpr int H = decltype(hc)::value;
        const uint8_t *img = lds + H * L::kStageBytes;
#pragma unroll
        for (int bb = 0; bb < 4; bb++) {
            const int b = 4 * H + bb;
            const int at = b * F::kBlockBytes + F::code_byte(kg);
            const uint32_t *wp = reinterpret_cast<const uint32_t *>(myrow + (at & ~3));
            uint32_t w[F::kWin], c[F::kWin - 1];
#pragma unroll
            for (int q = 0; q < F::kWin; q++) w[q] = wp[q];
#pragma unroll
            for (int q = 0; q < F::kWin - 1; q++) c[q] = (b & 1) ? w[q] : __builtin_amdgcn_alignbit(w[q + 1], w[q], 16);
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(myrow + b * F::kBlockBytes));
            const h8 f0 = F::frag(c, 0, magic), f1 = F::frag(c, 1, magic);
            const int o0 = F::octet(bb, kg, 0), o1 = F::octet(bb, kg, 1);  // octets of the half: 0 .. 15
            // (two tiles at a time and nothing moved across the pairs: with all four tiles' products in flight the kernel spills)
#pragma unroll
            for (int t0 = 0; t0 < NT; t0 += 2) {
                f16v p[2];
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const int t = t0 + u;
                    if (t >= NT) continue;
                    const h8 x0 = *reinterpret_cast<const h8 *>(img + t * G::kHalfBytes + (o0 * kMT + col) * 16);
                    const h8 x1 = *reinterpret_cast<const h8 *>(img + t * G::kHalfBytes + (o1 * kMT + col) * 16);
#pragma unroll
                    for (int r = 0; r < 16; r++) p[u][r] = 0.f;
                    p[u] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x0, f0, p[u], 0, 0, 0);
                    p[u] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x1, f1, p[u], 0, 0, 0);
                }
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const int t = t0 + u;
                    if (t >= NT) continue;
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[t][r] = fmaf(d, p[u][r], acc[t][r]);
                    // (the sums are pinned here: left free, the multiply-adds drift to the end of the stretch and every block's
                    // products stay in registers until then - 192 registers for one tile, spills from two)
                    asm volatile("" : "+v"(acc[t]));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // issue order: stage(0,0) fetch(0) fetch(1) | per stretch j: stage(j,1) | stage(j+1,0) fetch(j+2)
    stage(0, 0);
    asm volatile("" ::: "memory");  // (the counted waits rely on this order of the requests)
    fetch(0);
    asm volatile("" ::: "memory");
    if (nst > 1) fetch(1);
    for (int j = 0; j < nst; j++) {
        // first half: its image and this wavefront's stretch must be there (the request of the next stretch, issued after both, may
        // still be out); every wavefront has finished with stage 1, which the second half's image now overwrites
        meet(j + 1 >= nst);
        stage(j, 1);
        const uint8_t *myrow = park0 + (j & 1) * kParkBytes + col * 144;
        half(std::integral_constant<int, 0>(), myrow);
        // second half: the image requested above is the youngest request
        meet(true);
        if (j + 1 < nst) stage(j + 1, 0);
        half(std::integral_constant<int, 1>(), myrow);
        // the stretch has been read out: its park takes the stretch after the next
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        if (j + 2 < nst) fetch(j + 2);
    }

    if (n < N) {
        // lane holds y[m = 32 t + 8 (r / 4) + 4 kg + r % 4][n] for its K-slice
#pragma unroll
        for (int t = 0; t < NT; t++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + 32 * t + 8 * (r >> 2) + 4 * kg + (r & 3);
                if (m < M) partial[((int64_t)slice * M + m) * N + n] = acc[t][r];
            }
        }
    }
}

// ---- Q8_0 at more than 32 batch rows -------------------------------------------------------------------------------
//
// The same ring of half images and the same contraction as mmq_b32_tiles_kernel.  A Q8_0 stretch is 272 bytes of a row
// (8.5 KiB per tile of 32 rows): two parked tiles per wavefront do not fit beside the ring, so a wavefront has ONE park and
// the next stretch travels through registers, as in mmq_b32_kernel - requested when the stretch before it has been stored to
// the park, stored when that one has been read out.  Request order per stretch j: stage(j,1), loads(j+1) | stage(j+1,0); the
// wait in front of the second half leaves the nine register loads of the next stretch in flight.
template <int NT> struct Q8TilesOf {
    typedef B32Geom<kQ8_0> G;
    static constexpr int kStageBytes = NT * Q4KTiles::kHalfBytes;
    static constexpr int kRingBytes = 2 * kStageBytes;
    static constexpr int kLds = kRingBytes + Q4KTiles::kWaves * G::kWaveLds;  // (kWaveLds carries the slack for a code window that ends past the last row)
    static_assert(kLds <= 160 * 1024, "images + parked tiles exceed LDS");
};

template <int NT>
__global__ __launch_bounds__(64 * Q4KTiles::kWaves) void mmq_q8_tiles_kernel(const uint8_t *__restrict__ ximg, const uint8_t *__restrict__ W0,
                                                                              float *__restrict__ partial0, int M, int K, int N, int64_t row_bytes, int S,
                                                                              int m0, const uint8_t *__restrict__ W2, float *__restrict__ partial2) {
    typedef B32<kQ8_0> F;
    typedef B32Geom<kQ8_0> G;
    typedef Q4KTiles Q;
    typedef Q8TilesOf<NT> L;
    static_assert(G::kLoads == 9, "the counted wait below assumes nine load instructions per stretch");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint8_t *__restrict__ W = blockIdx.z ? W2 : W0;
    float *__restrict__ partial = blockIdx.z ? partial2 : partial0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 5, col = lane & 31;
    const int slice = blockIdx.y, nslices = gridDim.y;
    const int per_slice = S >> 8, first = slice * per_slice;
    const int nst = min(per_slice, (K >> 8) - first);  // stretches of this slice (at least one)
    const int row0 = (int)blockIdx.x * Q::kRows + wave * 32;
    const int n = row0 + col;  // this lane's weight row

    // chunk c = lane + 64 i of a stretch is chunk c % kCPR of row c / kCPR of the tile (rows past N re-read the last one)
    uint32_t coff[G::kLoads];
#pragma unroll
    for (int i = 0; i < G::kLoads; i++) {
        const int c = min(lane + 64 * i, G::kChunks - 1);
        coff[i] = (uint32_t)min(c / G::kCPR, max(N - 1 - row0, 0)) * (uint32_t)row_bytes + (uint32_t)(c % G::kCPR) * 16u;
    }
    const uint8_t *wtile = W + (int64_t)min(row0, N - 1) * row_bytes + (int64_t)first * G::kStretchBytes;
    typedef uint32_t Chunk __attribute__((ext_vector_type(4)));
    typedef Chunk ChunkA4 __attribute__((aligned(4)));  // (rows are 4-byte aligned in general)
    Chunk buf[G::kLoads];
    auto load = [&](int j) __attribute__((always_inline)) {  // stretch j of the slice -> registers: exactly kLoads load instructions
        const uint8_t *base = wtile + (int64_t)j * G::kStretchBytes;
#pragma unroll
        for (int l = 0; l < G::kLoads; l++) buf[l] = *reinterpret_cast<const ChunkA4 *>(base + coff[l]);
    };
    uint8_t *const park = lds + L::kRingBytes + wave * G::kWaveLds;
    const uint8_t *const myrow = park + col * G::kStretchBytes;

    const size_t img_bytes = (size_t)S * 64;
    const uint8_t *img0 = ximg + ((size_t)(m0 / kMT) * nslices + slice) * img_bytes;
    const size_t tile_stride = (size_t)nslices * img_bytes;
    auto stage = [&](int j, int h) __attribute__((always_inline)) {  // half h (four blocks) of stretch j of every tile -> ring stage h
        uint8_t *dst = lds + h * L::kStageBytes;
        for (int i = wave; i < NT * 8; i += Q::kWaves) {
            const int t = i >> 3, ck = i & 7;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void *)(img0 + t * tile_stride + j * 16384 + h * Q::kHalfBytes + ck * 1024 + lane * 16),
                (__attribute__((address_space(3))) void *)(dst + t * Q::kHalfBytes + ck * 1024), 16, 0, 0);
        }
    };
    auto meet = [&](bool all) __attribute__((always_inline)) {  // (see mmq_q4k_tiles_kernel)
        if (all) __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        else __builtin_amdgcn_s_waitcnt(0x0F79);       // vmcnt(9)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    f16v acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[t][r] = 0.f;
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));

    auto half = [&](auto hc) __attribute__((always_inline)) {  // four blocks of the parked stretch against ring stage H (as in mmq_b32_tiles_kernel)
        constexpr int H = decltype(hc)::value;
        const uint8_t *img = lds + H * L::kStageBytes;
#pragma unroll
        for (int bb = 0; bb < 4; bb++) {
            const int b = 4 * H + bb;
            const int at = b * F::kBlockBytes + F::code_byte(kg);
            const uint32_t *wp = reinterpret_cast<const uint32_t *>(myrow + (at & ~3));
            uint32_t w[F::kWin], c[F::kWin - 1];
#pragma unroll
            for (int q = 0; q < F::kWin; q++) w[q] = wp[q];
#pragma unroll
            for (int q = 0; q < F::kWin - 1; q++) c[q] = (b & 1) ? w[q] : __builtin_amdgcn_alignbit(w[q + 1], w[q], 16);
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(myrow + b * F::kBlockBytes));
            const h8 f0 = F::frag(c, 0, magic), f1 = F::frag(c, 1, magic);
            const int o0 = F::octet(bb, kg, 0), o1 = F::octet(bb, kg, 1);  // octets of the half: 0 .. 15
#pragma unroll
            for (int t0 = 0; t0 < NT; t0 += 2) {
                f16v p[2];
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const int t = t0 + u;
                    if (t >= NT) continue;
                    const h8 x0 = *reinterpret_cast<const h8 *>(img + t * Q::kHalfBytes + (o0 * kMT + col) * 16);
                    const h8 x1 = *reinterpret_cast<const h8 *>(img + t * Q::kHalfBytes + (o1 * kMT + col) * 16);
#pragma unroll
                    for (int r = 0; r < 16; r++) p[u][r] = 0.f;
                    p[u] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x0, f0, p[u], 0, 0, 0);
                    p[u] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x1, f1, p[u], 0, 0, 0);
                }
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const int t = t0 + u;
                    if (t >= NT) continue;
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[t][r] = fmaf(d, p[u][r], acc[t][r]);
                    asm volatile("" : "+v"(acc[t]));  // (pinned: see mmq_b32_tiles_kernel)
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    stage(0, 0);
    asm volatile("" ::: "memory");  // (the counted wait relies on the order of the requests)
    load(0);
    for (int j = 0; j < nst; j++) {
        // first half: its image and this wavefront's stretch (in registers) must be there; every wavefront has finished with stage 1
        meet(true);
        stage(j, 1);
        asm volatile("" ::: "memory");
        // park the stretch (LDS operations of one wavefront execute in order; no other wavefront reads it)
#pragma unroll
        for (int l = 0; l < G::kLoads; l++)
            if (lane + 64 * l < G::kChunks) *reinterpret_cast<Chunk *>(park + (lane + 64 * l) * 16) = buf[l];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const bool more = j + 1 < nst;
        if (more) load(j + 1);
        asm volatile("" ::: "memory");
        half(std::integral_constant<int, 0>());
        // second half: the image requested above must be there; the register loads of the next stretch, issued after it, may still be out
        meet(!more);
        if (more) stage(j + 1, 0);
        half(std::integral_constant<int, 1>());
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the reads above are done before the next stretch is parked
        __builtin_amdgcn_wave_barrier();
    }

    if (n < N) {
        // lane holds y[m = 32 t + 8 (r / 4) + 4 kg + r % 4][n] for its K-slice
#pragma unroll
        for (int t = 0; t < NT; t++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + 32 * t + 8 * (r >> 2) + 4 * kg + (r & 3);
                if (m < M) partial[((int64_t)slice * M + m) * N + n] = acc[t][r];
            }
        }
    }
}

template <int T, int RT>
int launch_mmq_b32(const void *x, bool x_is_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y, hipStream_t s,
                   const MmqExtra *ex) {
    const uint8_t *W2 = ex ? ex->W2 : nullptr;
    const RmsNorm *norm = ex ? ex->norm : nullptr;
    const int cus = device_cu_count();
    const int mtiles = (int)((M + kMT - 1) / kMT);
    // more than 32 batch rows: the kernels that walk up to four tiles of 32 rows per launch (Q8_0 has its own, with one parked tile)
    constexpr bool kHasTiles = true;
    constexpr bool kDmaTiles = B32<T>::kBlockBytes == 18;
    // (where its 256-row workgroups with the shortest slices still cover three quarters of the CUs: on 4096 x 4096 they are 128, and
    // the kernel below it stays ahead from 128 rows on, 26 against 32 us)
    const bool together = kHasTiles && mtiles >= 2 && tiles_together_mode() != 0 &&
                          ((N + Q4KTiles::kRows - 1) / Q4KTiles::kRows) * ((K + 511) / 512) * (W2 ? 2 : 1) >= (int64_t)cus * 3 / 4;
    const int64_t rowwgs = together ? (N + Q4KTiles::kRows - 1) / Q4KTiles::kRows : (N + 32 * RT - 1) / (32 * RT);
    // slices of 1024 when that still leaves every CU a workgroup and a half (LDS holds a 1024-value image
    // next to the parked stretches, not a 2048-value one); the kernel for several tiles has one workgroup per CU at a time
    // and takes the long slices from three quarters of the CUs on
    const int S = together ? (rowwgs * ((K + 1023) / 1024) * (W2 ? 2 : 1) >= (int64_t)cus * 3 / 4 ? 1024 : 512)
                           : (rowwgs * ((K + 1023) / 1024) * mtiles >= (int64_t)cus * 3 / 2 ? 1024 : 512);
    const int nslices = (int)((K + S - 1) / S);
    const size_t lds_bytes = (size_t)S * 64 + (size_t)2 * RT * B32Geom<T>::kWaveLds;  // image (later the handed-over tiles) + parked stretches
    static const bool lds_ok = [] {
        return hipFuncSetAttribute(reinterpret_cast<const void *>(mmq_b32_kernel<T, RT>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   1024 * 64 + 2 * RT * B32Geom<T>::kWaveLds) == hipSuccess;
    }();
    if (!lds_ok) return fail(GQ_ERR_HIP, "mmq: cannot reserve %d bytes of LDS", 1024 * 64 + 2 * RT * B32Geom<T>::kWaveLds);
    // workspace: [activation images: mtiles x nslices x S x 64 bytes][slice scales: nslices x M][partial sums: nslices x M x N fp32,
    // twice for a gated pair]
    const size_t img_bytes = (size_t)mtiles * nslices * S * 64;
    const size_t part_bytes = (size_t)nslices * M * N * sizeof(float);
    void *ws = nullptr;
    if (int rc = stream_workspace(s, img_bytes + mmq_scale_bytes(nslices, M) + part_bytes * (W2 ? 2 : 1), &ws)) return rc;
    uint8_t *ximg = reinterpret_cast<uint8_t *>(ws);
    float *xscale = reinterpret_cast<float *>(ximg + img_bytes);
    float *partial = reinterpret_cast<float *>(ximg + img_bytes + mmq_scale_bytes(nslices, M));
    const int64_t row_bytes = (K / 32) * B32<T>::kBlockBytes;
    const dim3 xgrid((unsigned)(mtiles * nslices * 4));
    auto prep = [&](auto kernel) {
        return launch(kernel, xgrid, dim3(256), 0, s, x, ximg, xscale, (int)M, (int)K, S, nslices, norm ? norm->gain : nullptr, norm ? norm->gain_offset : 0.f,
                      norm ? mmq_xss(xscale, nslices, M) : nullptr);
    };
    if (int rc = x_is_bf16 ? prep(mmq_b32_xprep_kernel<true>) : prep(mmq_b32_xprep_kernel<false>)) return rc;
    float *partial2 = W2 ? partial + (size_t)nslices * M * N : nullptr;
    if constexpr (kHasTiles) {
        if (together) {
            static const bool tiles_lds_ok = [] {
                auto room = [](auto kernel, int bytes) {
                    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess;
                };
                if constexpr (kDmaTiles)
                    return room(mmq_b32_tiles_kernel<T, 1>, B32TilesOf<1>::kLds) && room(mmq_b32_tiles_kernel<T, 2>, B32TilesOf<2>::kLds) &&
                           room(mmq_b32_tiles_kernel<T, 3>, B32TilesOf<3>::kLds) && room(mmq_b32_tiles_kernel<T, 4>, B32TilesOf<4>::kLds);
                else
                    return room(mmq_q8_tiles_kernel<1>, Q8TilesOf<1>::kLds) && room(mmq_q8_tiles_kernel<2>, Q8TilesOf<2>::kLds) &&
                           room(mmq_q8_tiles_kernel<3>, Q8TilesOf<3>::kLds) && room(mmq_q8_tiles_kernel<4>, Q8TilesOf<4>::kLds);
            }();
            if (!tiles_lds_ok) return fail(GQ_ERR_HIP, "mmq: cannot reserve %d bytes of LDS", kDmaTiles ? B32TilesOf<4>::kLds : Q8TilesOf<4>::kLds);
            const dim3 tgrid((unsigned)rowwgs, (unsigned)nslices, W2 ? 2u : 1u);
            // (the tiles are dealt evenly over the fewest launches, as for Q4_K)
            const int nlaunch = (mtiles + Q4KTiles::kMaxTiles - 1) / Q4KTiles::kMaxTiles;
            for (int l = 0, tile0 = 0; l < nlaunch; l++) {
                const int ntile = (mtiles - tile0 + (nlaunch - l) - 1) / (nlaunch - l);
                const int64_t m0 = (int64_t)tile0 * kMT;
                tile0 += ntile;
                auto go = [&](auto kernel, int lds) {
                    return launch(kernel, tgrid, dim3(64 * Q4KTiles::kWaves), (size_t)lds, s, (const uint8_t *)ximg, W, partial, (int)M, (int)K, (int)N,
                                  row_bytes, S, (int)m0, W2, partial2);
                };
                int rc;
                if constexpr (kDmaTiles)
                    rc = ntile == 4   ? go(mmq_b32_tiles_kernel<T, 4>, B32TilesOf<4>::kLds)
                         : ntile == 3 ? go(mmq_b32_tiles_kernel<T, 3>, B32TilesOf<3>::kLds)
                         : ntile == 2 ? go(mmq_b32_tiles_kernel<T, 2>, B32TilesOf<2>::kLds)
                                      : go(mmq_b32_tiles_kernel<T, 1>, B32TilesOf<1>::kLds);
                else
                    rc = ntile == 4   ? go(mmq_q8_tiles_kernel<4>, Q8TilesOf<4>::kLds)
                         : ntile == 3 ? go(mmq_q8_tiles_kernel<3>, Q8TilesOf<3>::kLds)
                         : ntile == 2 ? go(mmq_q8_tiles_kernel<2>, Q8TilesOf<2>::kLds)
                                      : go(mmq_q8_tiles_kernel<1>, Q8TilesOf<1>::kLds);
                if (rc) return rc;
            }
            return launch_mmq_reduce(partial, partial2, xscale, nslices, M, K, N, bias, act, y, ex, s);
        }
    }
    const dim3 grid((unsigned)rowwgs, (unsigned)nslices, (unsigned)mtiles * (W2 ? 2u : 1u));  // (both matrices of a gated pair in one launch)
    if (int rc = launch(mmq_b32_kernel<T, RT>, grid, dim3(RT * 128), lds_bytes, s, (const uint8_t *)ximg, W, partial, (int)M, (int)K, (int)N, row_bytes, S,
                        mtiles, W2, partial2))
        return rc;
    return launch_mmq_reduce(partial, partial2, xscale, nslices, M, K, N, bias, act, y, ex, s);
}


// ---- small batches of Q6_K --------------------------------------------------------------------------
//
// Same plan again.  A super-block is 210 bytes (2 bytes off a dword boundary every other one), so a
// wavefront's unit is a PAIR of super-blocks: 420 bytes = 105 dwords per row, dword-aligned when K
// is a multiple of 512.  The wavefront reads the pair of its 32 rows as consecutive dwords
// (coalesced), parks it in its private piece of LDS (row stride 105 dwords: odd, conflict-free) and
// lane (col = lane % 32, kg = lane / 32) picks row col's codes out of it.  One MFMA (K = 16) is
// exactly one 16-value scale group: lane kg holds values 8 kg .. 8 kg + 7 of it, assembled from the
// low nibbles / high bit pairs into bytes, turned into exact fp16 integers code - 32, and the
// group's partial tile is scaled by d * sc in fp32.
// Slices are 1024 values (two pairs: one per wavefront of a row tile); RT = 4 row tiles per workgroup (2 for problems
// that would not give every CU a workgroup otherwise).
// A wavefront parks its pair one super-block at a time (dwords 0 .. 52 of the pair, then dwords 52 .. 104: the
// second super-block starts 2 bytes into dword 52), so that the 64 KiB activation image and the parked halves of
// EIGHT wavefronts fit LDS: with two wavefronts per SIMD one's arithmetic hides the other's LDS and memory waits
// (four wavefronts parking whole pairs left every SIMD a single wavefront: 43 us on 4096 -> 14336 at 8 rows).
constexpr int kQ6PairBytes = 420;
constexpr int kQ6HalfDwords = 53, kQ6HalfBytes = 4 * kQ6HalfDwords;  // 212 bytes per row (odd dword stride: conflict-free)
constexpr int kQ6Loads = (32 * kQ6HalfDwords + 63) / 64;  // 27 dword loads per lane and half (the last: half a wavefront)
constexpr int kQ6WaveLds = 32 * kQ6HalfBytes + 16;         // + slack for a window that ends past the last row
constexpr int kQ6Slice = 1024;

// two dwords holding the 8 bytes at byte offset `at` of the parked row (at % 4 is 0 or 2, known at compile time)
__device__ __forceinline__ void q6_bytes8(const uint8_t *row, int at, uint32_t &a, uint32_t &b) {
    const uint32_t *p = reinterpret_cast<const uint32_t *>(row + (at & ~3));
    if (at & 2) {
        const uint32_t w0 = p[0], w1 = p[1], w2 = p[2];
        a = __builtin_amdgcn_alignbit(w1, w0, 16);
        b = __builtin_amdgcn_alignbit(w2, w1, 16);
    } else {
        a = p[0];
        b = p[1];
    }
}

// (Launched with RT * 128 threads, RT = 2 or 4 row tiles.  Declared for up to 512: with a bound of 256 the compiler puts every MFMA
// result into accumulation registers and copies it back out, 16 extra instructions per MFMA.)
template <int RT>
__global__ __launch_bounds__(512) void mmq_q6k_kernel(const uint8_t *__restrict__ ximg, const uint8_t *__restrict__ W,
                                                              float *__restrict__ partial0, int M, int K, int N, int64_t row_bytes, int mtiles,
                                                              const uint8_t *__restrict__ W2, float *__restrict__ partial2) {
    const bool second = (int)blockIdx.z >= mtiles;  // the second matrix of a gated pair
    const uint8_t *__restrict__ Wm = second ? W2 : W;
    float *__restrict__ partial = second ? partial2 : partial0;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kg = lane >> 5, col = lane & 31;
    const int rt = wave % RT, par = wave / RT;
    const int slice = blockIdx.y, nslices = gridDim.y, mt = second ? (int)blockIdx.z - mtiles : (int)blockIdx.z;
    constexpr int img_bytes = kQ6Slice * 64;
    const int kpairs = K >> 9;                                  // pairs of a row
    const int n0 = (blockIdx.x * RT + rt) * 32;              // first W row of this wavefront's tile
    uint8_t *park = lds + img_bytes + wave * kQ6WaveLds;

    // the slice's activation image goes straight from global memory into LDS (no registers)
    {
        const uint8_t *img = ximg + ((size_t)mt * nslices + slice) * img_bytes;
        for (int i = wave; i < img_bytes / 1024; i += 2 * RT)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(img + i * 1024 + lane * 16),
                                             (__attribute__((address_space(3))) void *)(lds + i * 1024), 16, 0, 0);
    }
    // This wavefront's pair of the slice (a pair beyond K re-reads the row's last one: its activations
    // are zero in the image), one half at a time.  Dword lane + 64 i of a half tile is dword d % 53 of row d / 53.
    const uint8_t *pair = Wm + (int64_t)min(n0, N - 1) * row_bytes + (int64_t)min(2 * slice + par, kpairs - 1) * kQ6PairBytes;
    const int rows_left = max(N - 1 - n0, 0);
    auto park_half = [&](int sbp) __attribute__((always_inline)) {
        uint32_t v[kQ6Loads];
#pragma unroll
        for (int i = 0; i < kQ6Loads; i++) {
            const int d = min(lane + 64 * i, 32 * kQ6HalfDwords - 1);
            v[i] = *reinterpret_cast<const uint32_t *>(pair + (int64_t)min(d / kQ6HalfDwords, rows_left) * row_bytes +
                                                       (sbp * (kQ6HalfDwords - 1) + d % kQ6HalfDwords) * 4);
        }
#pragma unroll
        for (int i = 0; i < kQ6Loads; i++)
            if (lane + 64 * i < 32 * kQ6HalfDwords) reinterpret_cast<uint32_t *>(park)[lane + 64 * i] = v[i];
    };
    park_half(0);
    // a barrier does not wait for loads in flight: every wavefront's share of the image copy must have landed first
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // image landed; the parked half is this wavefront's own

    f16v acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));
    const h2 off = as_h2(0xE420E420u);  // (-1056, -1056) = -(1024 + 32)
    const uint8_t *myrow = park + col * kQ6HalfBytes;
#pragma unroll
    for (int sbp = 0; sbp < 2; sbp++) {
        if (sbp == 1) {
            // (LDS operations of one wavefront execute in order; no other wavefront touches its parked half)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            park_half(1);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        const int b0 = sbp * 2;                      // byte offset of the super-block in the parked row
        const int sbg = 2 * par + sbp;               // super-block within the slice
        const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(myrow + b0 + 208));
#pragma unroll
        for (int h = 0; h < 2; h++) {
            // the half's eight scales (int8), 2 bytes off when sbp = 1
            uint32_t sc_lo, sc_hi;
            q6_bytes8(myrow, b0 + 192 + 8 * h, sc_lo, sc_hi);
#pragma unroll
            for (int is = 0; is < 2; is++) {
                uint32_t hq0, hq1;
                q6_bytes8(myrow, b0 + 128 + 32 * h + 16 * is + 8 * kg, hq0, hq1);
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    uint32_t lq0, lq1;
                    q6_bytes8(myrow, b0 + 64 * h + 32 * e + 16 * is + 8 * kg, lq0, lq1);
#pragma unroll
                    for (int nib = 0; nib < 2; nib++) {
                        const int qd = 2 * nib + e;  // quadrant of the half: values 32 qd + 16 is + 8 kg ..
                        const uint32_t c0 = ((lq0 >> (4 * nib)) & 0x0F0F0F0Fu) | (((hq0 >> (2 * qd)) & 0x03030303u) << 4);
                        const uint32_t c1 = ((lq1 >> (4 * nib)) & 0x0F0F0F0Fu) | (((hq1 >> (2 * qd)) & 0x03030303u) << 4);
                        uint4 o;  // fp16 pairs (0,2) (1,3) (4,6) (5,7) of code - 32
                        o.x = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, c0, 0x07020700u)) + off);
                        o.y = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, c0, 0x07030701u)) + off);
                        o.z = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, c1, 0x07020700u)) + off);
                        o.w = __builtin_bit_cast(uint32_t, as_h2(__builtin_amdgcn_perm(magic, c1, 0x07030701u)) + off);
                        const int oct = sbg * 32 + h * 16 + qd * 4 + is * 2 + kg;
                        const h8 xo = *reinterpret_cast<const h8 *>(lds + (oct * kMT + col) * 16);
                        f16v p;
#pragma unroll
                        for (int r = 0; r < 16; r++) p[r] = 0.f;
                        p = __builtin_amdgcn_mfma_f32_32x32x16_f16(xo, __builtin_bit_cast(h8, o), p, 0, 0, 0);
                        const int si = 2 * qd + is;  // scale index within the half
                        const int sc = (int)__builtin_amdgcn_sbfe((int)(si < 4 ? sc_lo : sc_hi), 8 * (si & 3), 8);  // (the builtin's result type is unsigned)
                        const float dsc = d * (float)sc;
#pragma unroll
                        for (int r = 0; r < 16; r++) acc[r] = fmaf(dsc, p[r], acc[r]);
                    }
                }
            }
        }
    }

    // the second wavefront of a row tile hands its 32 x 32 partial tile to the first through LDS
    __syncthreads();
    float *xch = reinterpret_cast<float *>(lds) + rt * (16 * 64);
    if (par > 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) xch[r * 64 + lane] = acc[r];
    }
    __syncthreads();
    const int n = n0 + col;
    if (par == 0 && n < N) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = mt * kMT + 8 * (r >> 2) + 4 * kg + (r & 3);
            if (m < M) partial[((int64_t)slice * M + m) * N + n] = acc[r] + xch[r * 64 + lane];
        }
    }
}

template <int RT>
int launch_mmq_q6k_rt(const MmqExtra *ex, const void *x, bool x_is_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
                   hipStream_t s) {
    constexpr int kLds = kQ6Slice * 64 + 2 * RT * kQ6WaveLds;
    static const bool lds_ok = [] {
        return hipFuncSetAttribute(reinterpret_cast<const void *>(mmq_q6k_kernel<RT>), hipFuncAttributeMaxDynamicSharedMemorySize, kLds) ==
               hipSuccess;
    }();
    if (!lds_ok) return fail(GQ_ERR_HIP, "mmq: cannot reserve %d bytes of LDS", kLds);
    const int mtiles = (int)((M + kMT - 1) / kMT);
    const int nslices = (int)((K + kQ6Slice - 1) / kQ6Slice);
    // workspace: [activation images: mtiles x nslices x 64 KiB][partial sums: nslices x M x N fp32, twice for a gated pair]
    const uint8_t *W2 = ex ? ex->W2 : nullptr;
    const RmsNorm *norm = ex ? ex->norm : nullptr;
    const size_t img_bytes = (size_t)mtiles * nslices * kQ6Slice * 64;
    const size_t part_bytes = (size_t)nslices * M * N * sizeof(float);
    void *ws = nullptr;
    if (int rc = stream_workspace(s, img_bytes + mmq_scale_bytes(nslices, M) + part_bytes * (W2 ? 2 : 1), &ws)) return rc;
    uint8_t *ximg = reinterpret_cast<uint8_t *>(ws);
    float *xscale = reinterpret_cast<float *>(ximg + img_bytes);
    float *partial = reinterpret_cast<float *>(ximg + img_bytes + mmq_scale_bytes(nslices, M));
    const int64_t row_bytes = (K / 256) * 210;
    const dim3 xgrid((unsigned)(mtiles * nslices * 4));
    auto prep = [&](auto kernel) {
        return launch(kernel, xgrid, dim3(256), 0, s, x, ximg, xscale, (int)M, (int)K, kQ6Slice, nslices, norm ? norm->gain : nullptr,
                      norm ? norm->gain_offset : 0.f, norm ? mmq_xss(xscale, nslices, M) : nullptr);
    };
    if (int rc = x_is_bf16 ? prep(mmq_b32_xprep_kernel<true>) : prep(mmq_b32_xprep_kernel<false>)) return rc;
    const dim3 grid((unsigned)((N + 32 * RT - 1) / (32 * RT)), (unsigned)nslices, (unsigned)mtiles * (W2 ? 2u : 1u));  // (a gated pair: one launch)
    float *partial2 = W2 ? partial + (size_t)nslices * M * N : nullptr;
    if (int rc = launch(mmq_q6k_kernel<RT>, grid, dim3(RT * 128), (size_t)kLds, s, (const uint8_t *)ximg, W, partial, (int)M, (int)K, (int)N,
                        row_bytes, mtiles, W2, partial2))
        return rc;
    return launch_mmq_reduce(partial, partial2, xscale, nslices, M, K, N, bias, act, y, ex, s);
}

// Four row tiles per workgroup (eight wavefronts) when that still gives every CU a workgroup, else two.
int launch_mmq_q6k(const MmqExtra *ex, const void *x, bool x_is_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
                   hipStream_t s) {
    const int64_t wgs4 = ((N + 127) / 128) * ((K + kQ6Slice - 1) / kQ6Slice) * ((M + kMT - 1) / kMT);
    return wgs4 >= device_cu_count() ? launch_mmq_q6k_rt<4>(ex, x, x_is_bf16, M, K, W, N, bias, act, y, s)
                                     : launch_mmq_q6k_rt<2>(ex, x, x_is_bf16, M, K, W, N, bias, act, y, s);
}

}  // namespace

bool mmq_supported(int type, int64_t M, int64_t K, int64_t N, const void *x, const void *bias, const void *y) {
    // K <= 2^26: the kernels address the 32 rows of a tile by 32-bit byte offsets from its first row (31 rows of at most
    // 2^26 * 34 / 32 bytes stay below 2^32)
    // (Q4_K walks four tiles of 32 rows per launch and stays ahead of the two-pass GEMM for longer than the others)
    const bool shape_ok = M >= 2 && M <= (type == kQ4_K ? 512 : 256) && N % 4 == 0 && N <= (int64_t)INT32_MAX / 2 && K <= ((int64_t)1 << 26) &&
                          ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(bias) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    if (type == kQ4_K) return shape_ok && K % 256 == 0;
    if (type == kQ8_0 || type == kQ4_0 || type == kIQ4_NL) return shape_ok && K % 256 == 0;  // whole stretches of 8 blocks
    if (type == kQ6_K) return shape_ok && K % 512 == 0;                   // whole, dword-aligned pairs of super-blocks
    return false;
}

namespace {
// GOMLX_HIPQ_COOP=1 sends the Q4_K split-K route through the kernel that stages the activations itself (two launches
// instead of three).  It is correct and tested, and it is slower: 24.0 against 20.5 us on a 14336 -> 4096 matrix at 32 rows,
// because a record travels workgroup -> memory -> flag -> other workgroups in four dependent trips to memory, longer than
// the pre-pass launch they replace; it stays selectable so that the comparison can be repeated.
// GOMLX_HIPQ_COOP_SPIN_TICKS=n bounds the wait for published activation records (100 MHz ticks; 0 makes every wait run
// out at once, which is how the tests reach the path that stages the missing records locally).  Both are read at every call.
bool coop_enabled() {
    const char *e = std::getenv("GOMLX_HIPQ_COOP");
    return e && e[0] == '1';
}
int coop_spin_ticks() {
    const char *e = std::getenv("GOMLX_HIPQ_COOP_SPIN_TICKS");
    const long v = e ? std::atol(e) : 20000;  // 200 us: a record is published a few microseconds into the kernel
    return v < 0 ? 0 : v > 100000000 ? 100000000 : (int)v;
}

// GOMLX_HIPQ_Q4K_TILES_TOGETHER=0: batches of more than 32 rows as one launch of mmq_q4k_kernel per 32 rows; =2: batches of up
// to 32 rows through mmq_q4k_tiles_kernel<1> as well (tuning runs and comparisons only).  Read at every call.
int tiles_together_mode() {
    const char *e = std::getenv("GOMLX_HIPQ_Q4K_TILES_TOGETHER");
    return e && e[0] >= '0' && e[0] <= '2' ? e[0] - '0' : 1;
}

// `count` Q4_K matrices against one activation image: the pre-pass once, every matrix's row ranges in one launch of the
// main kernel, one reduction.  A single matrix may carry the extras (gated pair, residual); a set carries a normalisation only.
int run_q4k_set(const void *x, bool x_is_bf16, int64_t M, int64_t K, int count, const MmqSetItem *items, const MmqExtra *ex, hipStream_t s) {
    const uint8_t *W2 = (ex && count == 1) ? ex->W2 : nullptr;
    typedef Q4KTile<kQ4KRowTiles> Tile;
    static const bool lds_ok = [] {
        return hipFuncSetAttribute(reinterpret_cast<const void *>(mmq_q4k_kernel<kQ4KRowTiles>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   Tile::kLds) == hipSuccess;
    }();
    if (!lds_ok) return fail(GQ_ERR_HIP, "mmq: cannot reserve %d bytes of LDS", Tile::kLds);
    const int mtiles = (int)((M + kMT - 1) / kMT);
    const int64_t sbs = K / 256;
    // more than 32 batch rows: the kernel that walks up to four tiles of 32 together (256 rows of W per workgroup)
    // (a single tile of up to 32 rows as well where the matrix is wide and large - 4096 -> 14336 at 32 rows 22.7 against 25.3 us,
    // the gated pair 35.8 against 37.5, a 128k-vocabulary head 134 against 143 - but not on long-K ones: 14336 -> 4096 23.7 against 20.5)
    int64_t all_rows = 0;
    for (int i = 0; i < count; i++) all_rows += items[i].N;
    const bool wide = all_rows >= 2 * K && all_rows * (K / 256) * 144 >= ((int64_t)24 << 20);
    const bool together = !coop_enabled() && (tiles_together_mode() == 2 || (tiles_together_mode() == 1 && (mtiles >= 2 || wide)));
    static const bool tiles_lds_ok = [] {
        auto room = [](auto kernel, int bytes) {
            return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess;
        };
        return room(mmq_q4k_tiles_kernel<1>, Q4KTilesOf<1>::kLds) && room(mmq_q4k_tiles_kernel<2>, Q4KTilesOf<2>::kLds) &&
               room(mmq_q4k_tiles_kernel<3>, Q4KTilesOf<3>::kLds) && room(mmq_q4k_tiles_kernel<4>, Q4KTilesOf<4>::kLds);
    }();
    if (together && !tiles_lds_ok) return fail(GQ_ERR_HIP, "mmq: cannot reserve %d bytes of LDS", Q4KTilesOf<4>::kLds);
    const int wg_rows = together ? Q4KTiles::kRows : Tile::kRows;
    Q4KSet set = {};
    MmqSetOut out = {};
    int64_t rowwgs = 0, N = 0;  // workgroups along the rows of all matrices; their columns side by side
    for (int i = 0; i < count; i++) {
        set.W[i] = items[i].W; set.N[i] = (int)items[i].N; set.wg0[i] = (int)rowwgs; set.n0[i] = (int)N;
        out.bias[i] = items[i].bias; out.y[i] = items[i].y; out.N[i] = (int)items[i].N; out.n0[i] = (int)N; out.act[i] = items[i].act;
        rowwgs += (items[i].N + wg_rows - 1) / wg_rows;
        N += items[i].N;
    }
    set.count = out.count = count;
    set.ntot = out.ntot = (int)N;
    // Super-blocks per K-slice (at most 7: the image shares LDS with the parked tiles): the count that needs the fewest
    // rounds of workgroups over the chip times the length of a round (+3: what a workgroup costs beyond its
    // super-blocks); ties go to the longer slice (fewer partial sums).
    int slice_sb = Tile::kMaxSliceSB;
    {
        const int64_t cus = device_cu_count(), z = W2 ? 2 : 1;
        int64_t best_cost = INT64_MAX;
        for (int ssb = Tile::kMaxSliceSB; ssb >= 2; ssb--) {
            const int64_t wgs = rowwgs * ((sbs + ssb - 1) / ssb) * z;
            const int64_t cost = ((wgs + cus - 1) / cus) * (ssb + 3);
            if (cost < best_cost) { best_cost = cost; slice_sb = ssb; }
        }
    }
    if (const char *e = std::getenv("GOMLX_HIPQ_Q4K_SLICE_SB")) {  // (tuning runs only)
        const int v = std::atoi(e);
        if (v >= 1 && v <= Tile::kMaxSliceSB) slice_sb = v;
    }
    const int nslices = (int)((sbs + slice_sb - 1) / slice_sb);
    const int64_t row_bytes = (K / 256) * 144;
    const RmsNorm *norm = ex ? ex->norm : nullptr;
    float *partial2 = nullptr;
    const dim3 grid((unsigned)rowwgs, (unsigned)nslices, W2 ? 2u : 1u);  // (both matrices of a gated pair in one launch)
    // Without a normalisation the main kernel stages the activations itself (mmq_q4k_coop_kernel): no pre-pass launch.  It
    // needs a publisher per super-block of a slice among the row workgroups, and its flags in the workspace's flag words.
    const int nflags = mtiles * nslices * kFlagsPerSlice;
    if (!norm && rowwgs >= slice_sb && (size_t)nflags * sizeof(uint32_t) <= kWsSyncBytes && coop_enabled()) {
        typedef Q4KCoopTile<kQ4KRowTiles> CTile;
        static const bool coop_lds_ok = [] {
            return hipFuncSetAttribute(reinterpret_cast<const void *>(mmq_q4k_coop_kernel<kQ4KRowTiles, false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, CTile::kLds) == hipSuccess &&
                   hipFuncSetAttribute(reinterpret_cast<const void *>(mmq_q4k_coop_kernel<kQ4KRowTiles, true>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, CTile::kLds) == hipSuccess;
        }();
        if (!coop_lds_ok) return fail(GQ_ERR_HIP, "mmq: cannot reserve %d bytes of LDS", CTile::kLds);
        // workspace: [activation records: mtiles x nslices x 7 x kRecStride][partial sums: nslices x M x N fp32, twice for a gated pair]
        const size_t rec_bytes = (size_t)mtiles * nslices * CTile::kMaxSliceSB * kRecStride;
        const size_t part_bytes = (size_t)nslices * M * N * sizeof(float);
        void *ws = nullptr;
        uint32_t *flags = nullptr;
        if (int rc = stream_workspace(s, rec_bytes + part_bytes * (W2 ? 2 : 1), &ws, 0, &flags)) return rc;
        uint8_t *ximg = reinterpret_cast<uint8_t *>(ws);
        float *partial = reinterpret_cast<float *>(ximg + rec_bytes);
        partial2 = W2 ? partial + (size_t)nslices * M * N : nullptr;
        const int spin = coop_spin_ticks();
        for (int64_t m0 = 0; m0 < M; m0 += kMT) {
            const int rc = x_is_bf16 ? launch(mmq_q4k_coop_kernel<kQ4KRowTiles, true>, grid, dim3(64 * CTile::kWaves), (size_t)CTile::kLds, s, x, ximg,
                                              flags, set, partial, (int)M, (int)K, row_bytes, (int)m0, slice_sb, W2, partial2, spin)
                                     : launch(mmq_q4k_coop_kernel<kQ4KRowTiles, false>, grid, dim3(64 * CTile::kWaves), (size_t)CTile::kLds, s, x, ximg,
                                              flags, set, partial, (int)M, (int)K, row_bytes, (int)m0, slice_sb, W2, partial2, spin);
            if (rc) return rc;
        }
        if (count == 1)
            return launch_mmq_reduce(partial, partial2, nullptr, nslices, M, K, N, items[0].bias, items[0].act, items[0].y, ex, s, flags, nflags);
        const int64_t quads = M * N / 4;
        const int threads = quads / 256 >= 2 * device_cu_count() ? 256 : 64;
        return launch(mmq_reduce_set_kernel, dim3((unsigned)((quads + threads - 1) / threads)), dim3(threads), 0, s, (const float *)partial, nslices,
                      (int)M, out, (const float *)nullptr, (const float *)nullptr, 0.f, 1.0f / (float)K, flags, nflags);
    }
    // workspace: [activation images: mtiles x nslices x kLdsBytes][slice scales: nslices x M][partial sums: nslices x M x N fp32,
    // twice for a gated pair]
    const size_t img_bytes = (size_t)mtiles * nslices * kLdsBytes;
    const size_t part_bytes = (size_t)nslices * M * N * sizeof(float);
    void *ws = nullptr;
    if (int rc = stream_workspace(s, img_bytes + mmq_scale_bytes(nslices, M) + part_bytes * (W2 ? 2 : 1), &ws)) return rc;
    uint8_t *ximg = reinterpret_cast<uint8_t *>(ws);
    float *xscale = reinterpret_cast<float *>(ximg + img_bytes);
    float *partial = reinterpret_cast<float *>(ximg + img_bytes + mmq_scale_bytes(nslices, M));
    // (each workgroup of the pre-pass converts 2 or 4 of a tile's 32 columns: the finer split while it still leaves CUs idle)
    const bool fine = (int64_t)nslices * mtiles * 8 * 2 <= device_cu_count();
    const dim3 pgrid((unsigned)nslices, (unsigned)mtiles, fine ? 16u : 8u);
    const float *gain = norm ? norm->gain : nullptr;
    const float goff = norm ? norm->gain_offset : 0.f;
    float *xss = norm ? mmq_xss(xscale, nslices, M) : nullptr;
    auto prep = [&](auto kernel) { return launch(kernel, pgrid, dim3(512), 0, s, x, ximg, xscale, (int)M, (int)K, slice_sb, gain, goff, xss); };
    if (int rc = x_is_bf16 ? (fine ? prep(mmq_xprep_kernel<true, 1>) : prep(mmq_xprep_kernel<true, 2>))
                           : (fine ? prep(mmq_xprep_kernel<false, 1>) : prep(mmq_xprep_kernel<false, 2>)))
        return rc;
    partial2 = W2 ? partial + (size_t)nslices * M * N : nullptr;
    // (the tiles are dealt evenly over the fewest launches: five tiles go as 3 + 2, not as 4 + 1 - every launch streams all of W)
    const int nlaunch = (mtiles + Q4KTiles::kMaxTiles - 1) / Q4KTiles::kMaxTiles;
    for (int l = 0, tile0 = 0; together && l < nlaunch; l++) {
        const int ntile = (mtiles - tile0 + (nlaunch - l) - 1) / (nlaunch - l);
        const int64_t m0 = (int64_t)tile0 * kMT;
        tile0 += ntile;
        auto go = [&](auto kernel, int lds_bytes) {
            return launch(kernel, grid, dim3(64 * Q4KTiles::kWaves), (size_t)lds_bytes, s, (const uint8_t *)ximg, set, partial, (int)M, (int)K, row_bytes,
                          (int)m0, W2, partial2);
        };
        if (int rc = ntile == 4   ? go(mmq_q4k_tiles_kernel<4>, Q4KTilesOf<4>::kLds)
                     : ntile == 3 ? go(mmq_q4k_tiles_kernel<3>, Q4KTilesOf<3>::kLds)
                     : ntile == 2 ? go(mmq_q4k_tiles_kernel<2>, Q4KTilesOf<2>::kLds)
                                  : go(mmq_q4k_tiles_kernel<1>, Q4KTilesOf<1>::kLds))
            return rc;
    }
    for (int64_t m0 = 0; !together && m0 < M; m0 += kMT) {
        if (int rc = launch(mmq_q4k_kernel<kQ4KRowTiles>, grid, dim3(64 * Tile::kWaves), (size_t)Tile::kLds, s, (const uint8_t *)ximg, set, partial,
                            (int)M, (int)K, row_bytes, (int)m0, slice_sb, W2, partial2))
            return rc;
    }
    if (count == 1) return launch_mmq_reduce(partial, partial2, xscale, nslices, M, K, N, items[0].bias, items[0].act, items[0].y, ex, s);
    const int64_t quads = M * N / 4;
    const int threads = quads / 256 >= 2 * device_cu_count() ? 256 : 64;
    return launch(mmq_reduce_set_kernel, dim3((unsigned)((quads + threads - 1) / threads)), dim3(threads), 0, s, (const float *)partial, nslices, (int)M,
                  out, (const float *)xscale, (const float *)xss, norm ? norm->eps : 0.f,
                  1.0f / (float)K, (uint32_t *)nullptr, 0);
}
}  // namespace

int launch_mmq(int type, const void *x, bool x_is_bf16, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias,
               int act, float *y, hipStream_t s, const MmqExtra *ex) {
    // (four row tiles per workgroup measured a little faster than two)
    if (type == kQ8_0) return launch_mmq_b32<kQ8_0, 4>(x, x_is_bf16, M, K, W, N, bias, act, y, s, ex);
    if (type == kQ4_0) return launch_mmq_b32<kQ4_0, 4>(x, x_is_bf16, M, K, W, N, bias, act, y, s, ex);
    if (type == kIQ4_NL) return launch_mmq_b32<kIQ4_NL, 4>(x, x_is_bf16, M, K, W, N, bias, act, y, s, ex);
    if (type == kQ6_K) return launch_mmq_q6k(ex, x, x_is_bf16, M, K, W, N, bias, act, y, s);
    if (type != kQ4_K) return fail(GQ_ERR_NOT_IMPLEMENTED, "mmq: ggml type %d is not implemented", type);
    const MmqSetItem one{W, N, bias, act, y};
    return run_q4k_set(x, x_is_bf16, M, K, 1, &one, ex, s);
}

bool mmq_set_supported(int type, int count, const MmqSetItem *items, int64_t M, int64_t K, const void *x) {
    if (type != kQ4_K || count < 2 || count > kMaxSet) return false;
    int64_t total = 0;
    for (int i = 0; i < count; i++) {
        if (!mmq_supported(type, M, K, items[i].N, x, items[i].bias, items[i].y)) return false;
        total += items[i].N;
    }
    return total <= (int64_t)INT32_MAX / 2;
}

int launch_mmq_set(int type, const void *x, bool x_is_bf16, int64_t M, int64_t K, int count, const MmqSetItem *items, const RmsNorm *norm,
                   hipStream_t s) {
    if (type != kQ4_K || count < 1 || count > kMaxSet) return fail(GQ_ERR_NOT_IMPLEMENTED, "mmq: a set of %d matrices of type %d is not implemented", count, type);
    const MmqExtra ex{nullptr, nullptr, nullptr, norm};
    return run_q4k_set(x, x_is_bf16, M, K, count, items, norm ? &ex : nullptr, s);
}

}  // namespace gq
