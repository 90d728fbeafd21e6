// Device-side decoding of GGML blocks (Q8_0, Q4_0, IQ4_NL, Q4_K) for gfx950.
//
// Arithmetic follows ml/ggml/dequant.go:58-136 of the reference (Q8_0, Q4_0, IQ4_NL) and
// the public GGML block_q4_K layout (Q4_K): every fp32 multiply / subtract is a separate,
// individually rounded operation.  This translation unit family is compiled with
// -ffp-contract=off, so `a * b - c` below never becomes a fused multiply-add.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gq {

constexpr int kQ4_0 = 2, kQ8_0 = 8, kQ4_K = 12, kQ6_K = 14, kIQ4_NL = 20;
constexpr int kActNone = 0, kActGelu = 1, kActRelu = 2, kActSilu = 3, kActHardSwish = 4, kActTanh = 5;

template <int T> struct Geom;
template <> struct Geom<kQ4_0> { static constexpr int bpb = 18, vpb = 32; };
template <> struct Geom<kQ8_0> { static constexpr int bpb = 34, vpb = 32; };
template <> struct Geom<kIQ4_NL> { static constexpr int bpb = 18, vpb = 32; };
template <> struct Geom<kQ4_K> { static constexpr int bpb = 144, vpb = 256; };
template <> struct Geom<kQ6_K> { static constexpr int bpb = 210, vpb = 256; };

// 16 bytes that are only guaranteed to be 2-byte aligned (Q4_0 / Q8_0 payloads start two
// bytes into an 18- or 34-byte block).  gfx950 global loads accept unaligned addresses, so
// this still compiles to a single global_load_dwordx4.
struct __attribute__((packed, aligned(2))) u128_a2 { uint32_t v[4]; };

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    const uint16_t b = (uint16_t)h;
    _Float16 v;
    __builtin_memcpy(&v, &b, 2);
    return (float)v;  // v_cvt_f32_f16: exact, subnormals included
}

__device__ __forceinline__ uint32_t load_u16(const uint8_t *p) {
    return *reinterpret_cast<const uint16_t *>(p);
}

// Byte j of v as an fp32 number (v_cvt_f32_ubyteN).  Inline asm keeps the compiler from
// re-deriving the byte with a separate bit-field extract.
__device__ __forceinline__ float ubyte0(uint32_t v) { float f; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ubyte1(uint32_t v) { float f; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ubyte2(uint32_t v) { float f; asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ubyte3(uint32_t v) { float f; asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(v)); return f; }
// byte n of v as a signed 8-bit integer, converted to float in one instruction (sub-dword operand select with sign extension)
__device__ __forceinline__ float sbyte0(uint32_t v) { float f; asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float sbyte1(uint32_t v) { float f; asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float sbyte2(uint32_t v) { float f; asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float sbyte3(uint32_t v) { float f; asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(f) : "v"(v)); return f; }

// Public GGML IQ4_NL code book (compute.IQ4NLLookupTable, ml/ggml/dequant.go:130).
__device__ __forceinline__ float iq4nl_value(uint32_t nib) {
    // Packed as int8 in four dwords; selected with a byte permute instead of a memory table.
    const uint32_t t0 = 0xBFAD9881u;  // -127 -104 -83 -65
    const uint32_t t1 = 0xF6EADDCFu;  // -49 -35 -22 -10
    const uint32_t t2 = 0x26190D01u;  // 1 13 25 38
    const uint32_t t3 = 0x71594535u;  // 53 69 89 113
    const uint32_t lo = (nib & 4) ? t1 : t0;
    const uint32_t hi = (nib & 4) ? t3 : t2;
    const uint32_t w = (nib & 8) ? hi : lo;
    const int32_t b = (int32_t)(int8_t)(w >> ((nib & 3) * 8));
    return (float)b;
}

// The 6-bit (scale, min) pair of sub-block j (0..7) of a Q4_K super-block whose twelve
// packed bytes are given as three little-endian dwords a = s[0..3], b = s[4..7], c = s[8..11].
__device__ __forceinline__ void q4k_scale_min(uint32_t a, uint32_t b, uint32_t c, int j, uint32_t &sc, uint32_t &mn) {
    const int sh = (j & 3) * 8;
    const uint32_t aj = a >> sh, bj = b >> sh, cj = c >> sh;
    if (j < 4) {
        sc = aj & 63u;
        mn = bj & 63u;
    } else {
        sc = (cj & 0x0Fu) | (((aj >> 6) & 3u) << 4);
        mn = ((cj >> 4) & 0x0Fu) | (((bj >> 6) & 3u) << 4);
    }
}

// Exact dequantisation of 16 consecutive values of one weight row:
// out[0..15] = w[16*i .. 16*i+15].  Bit-exact with the reference arithmetic.
template <int T>
__device__ __forceinline__ void dequant16(const uint8_t *__restrict__ row, int64_t i, float *out);

template <>
__device__ __forceinline__ void dequant16<kQ8_0>(const uint8_t *__restrict__ row, int64_t i, float *out) {
    const uint8_t *blk = row + (i >> 1) * 34;
    const float d = half_bits_to_float(load_u16(blk));
    const u128_a2 q = *reinterpret_cast<const u128_a2 *>(blk + 2 + 16 * (i & 1));
#pragma unroll
    for (int w = 0; w < 4; w++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int32_t v = (int32_t)(int8_t)(q.v[w] >> (8 * j));
            out[4 * w + j] = (float)v * d;  // ml/ggml/dequant.go:74
        }
    }
}

template <>
__device__ __forceinline__ void dequant16<kQ4_0>(const uint8_t *__restrict__ row, int64_t i, float *out) {
    const uint8_t *blk = row + (i >> 1) * 18;
    const float d = half_bits_to_float(load_u16(blk));
    const u128_a2 q = *reinterpret_cast<const u128_a2 *>(blk + 2);
    const int sh = (int)(i & 1) * 4;  // values 0..15: low nibbles, 16..31: high nibbles
#pragma unroll
    for (int w = 0; w < 4; w++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t nib = (q.v[w] >> (8 * j + sh)) & 0x0Fu;
            out[4 * w + j] = ((float)nib - 8.0f) * d;  // ml/ggml/dequant.go:108-112
        }
    }
}

template <>
__device__ __forceinline__ void dequant16<kIQ4_NL>(const uint8_t *__restrict__ row, int64_t i, float *out) {
    const uint8_t *blk = row + (i >> 1) * 18;
    const float d = half_bits_to_float(load_u16(blk));
    const u128_a2 q = *reinterpret_cast<const u128_a2 *>(blk + 2);
    const int sh = (int)(i & 1) * 4;
#pragma unroll
    for (int w = 0; w < 4; w++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t nib = (q.v[w] >> (8 * j + sh)) & 0x0Fu;
            out[4 * w + j] = iq4nl_value(nib) * d;  // ml/ggml/dequant.go:130-133
        }
    }
}

template <>
__device__ __forceinline__ void dequant16<kQ4_K>(const uint8_t *__restrict__ row, int64_t i, float *out) {
    const uint8_t *sb = row + (i >> 4) * 144;  // 16 runs of 16 values per super-block
    const int idx = (int)(i & 15);
    const int g = idx >> 2;         // group of 64 values sharing 32 code bytes
    const int h = (idx >> 1) & 1;   // 0: low nibbles (sub-block 2g), 1: high nibbles (2g+1)
    const int p = idx & 1;          // which 16 of the 32 code bytes
    const uint4 hd = *reinterpret_cast<const uint4 *>(sb);
    const float d = half_bits_to_float(hd.x & 0xFFFFu);
    const float dmin = half_bits_to_float(hd.x >> 16);
    uint32_t sc, mn;
    q4k_scale_min(hd.y, hd.z, hd.w, 2 * g + h, sc, mn);
    const float ds = d * (float)sc;
    const float dm = dmin * (float)mn;
    const uint4 q = *reinterpret_cast<const uint4 *>(sb + 16 + 32 * g + 16 * p);
    const uint32_t qq[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int w = 0; w < 4; w++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t nib = (qq[w] >> (8 * j + 4 * h)) & 0x0Fu;
            out[4 * w + j] = ds * (float)nib - dm;
        }
    }
}

// Q6_K super-block: 128 bytes ql (low 4 bits), 64 bytes qh (high 2 bits), 16 int8 scales, fp16 d
// (210 bytes, 2-byte aligned).  Run i of 16 values lies in half h = i / 8 of the block, quadrant
// qd = (i / 2) % 4 (which selects 32 of the 64 ql bytes, the nibble, and the 2-bit field of qh)
// and covers l = 16 (i % 2) .. + 15, i.e. one scale.  w = (d * scale) * (q - 32): the exact product
// has at most 24 significant bits, so the order of the multiplications does not matter.
template <>
__device__ __forceinline__ void dequant16<kQ6_K>(const uint8_t *__restrict__ row, int64_t i, float *out) {
    const uint8_t *sb = row + (i >> 4) * 210;
    const int r = (int)(i & 15);
    const int h = r >> 3, qd = (r >> 1) & 3, l0 = (r & 1) * 16;
    const u128_a2 ql = *reinterpret_cast<const u128_a2 *>(sb + 64 * h + 32 * (qd & 1) + l0);
    const u128_a2 qh = *reinterpret_cast<const u128_a2 *>(sb + 128 + 32 * h + l0);
    const int sc = (int)(int8_t)sb[192 + 8 * h + 2 * qd + (r & 1)];
    const float ds = half_bits_to_float(load_u16(sb + 208)) * (float)sc;
    const int nsh = (qd >> 1) * 4, hsh = 2 * qd;
#pragma unroll
    for (int w = 0; w < 4; w++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t lo = (ql.v[w] >> (8 * j + nsh)) & 0x0Fu;
            const uint32_t hi = (qh.v[w] >> (8 * j + hsh)) & 0x03u;
            out[4 * w + j] = ds * (float)((int)(lo | (hi << 4)) - 32);
        }
    }
}

// Epilogue of the fused op: activation.Apply formulas
// (ml/layers/activation/activation.go:161,195,222-243,274-286); Gelu is the exact erf form.
// Activations that are rounded to fp16 operands are first scaled by a power of two per batch row
// (split-K kernels: per row and K-slice), so that their largest magnitude lands in [512, 1024):
// whatever the range of the inputs, nothing overflows (a sum of 32 values stays below 32768) and
// nothing that matters next to the largest value falls into fp16's subnormals.  The results are
// multiplied by the inverse (exact).  Zero, tiny-subnormal and non-finite maxima mean no scaling.
__device__ __forceinline__ void pow2_scale(float amax, float &s, float &inv) {
    const int e = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xFFu);
    if (e >= 10 && e <= 254) {
        s = __builtin_bit_cast(float, (uint32_t)(263 - e) << 23);    // 2^(136 - e): amax * s in [2^9, 2^10)
        inv = __builtin_bit_cast(float, (uint32_t)(e - 9) << 23);    // 2^(e - 136)
    } else {
        s = 1.f;
        inv = 1.f;
    }
}
__device__ __forceinline__ float amax8(const float4 &a, const float4 &b) {
    return fmaxf(fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))),
                 fmaxf(fmaxf(fabsf(b.x), fabsf(b.y)), fmaxf(fabsf(b.z), fabsf(b.w))));
}
// maximum over a full wavefront (all 64 lanes active): within rows of 16 lanes by data-parallel
// permutes, then over the four rows through scalar reads
__device__ __forceinline__ float wave_max(float v) {
#define GQ_DPP_MAX(ctrl) v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, true)))
    GQ_DPP_MAX(0xB1);   // quad_perm [1,0,3,2]
    GQ_DPP_MAX(0x4E);   // quad_perm [2,3,0,1]
    GQ_DPP_MAX(0x141);  // row_half_mirror
    GQ_DPP_MAX(0x140);  // row_mirror
#undef GQ_DPP_MAX
    const int b = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// 16 bytes to memory, written through the caches: once the store is acknowledged (s_waitcnt vmcnt) every other workgroup
// of the chip that has not read the line before in this kernel reads the new bytes.
__device__ __forceinline__ void store_through(void *p, const uint4 &v) {
    typedef uint32_t Chunk __attribute__((ext_vector_type(4)));
    const Chunk c = {v.x, v.y, v.z, v.w};
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(p), "v"(c) : "memory");
}

__device__ __forceinline__ float apply_act(int act, float v) {
    switch (act) {
    case kActRelu: return fmaxf(v, 0.0f);
    case kActSilu: return v / (1.0f + __expf(-v));
    case kActHardSwish: return v * fminf(fmaxf(v * (1.0f / 6.0f) + 0.5f, 0.0f), 1.0f);
    case kActTanh: return tanhf(v);
    case kActGelu: return v * 0.5f * (1.0f + erff(v * 0.70710678118654752f));
    default: return v;
    }
}

// Sum over the 64 lanes of a wavefront; every lane receives the total.  The first four
// steps are DPP moves inside a row of 16 lanes, the last two cross rows.
__device__ __forceinline__ float wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // row_mirror
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

}  // namespace gq
