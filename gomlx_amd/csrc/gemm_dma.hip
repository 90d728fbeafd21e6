// Quantised Dense for batches of 17 rows and more, in two passes:
//   1. the weight matrix is dequantised once into a 16-bit [N, K] image in a workspace (exact
//      fp32 values, one rounding to the MFMA operand type: the same operand values the fused
//      kernel of gemm.hip builds tile by tile);
//   2. a plain 16-bit x 16-bit -> fp32 MFMA GEMM contracts it with the activations.
//
// The fused kernel converts a 128-row slab of W again for every 256 rows of activations, and on a
// SIMD those vector-ALU instructions do not overlap with its MFMAs; it is cheaper to convert once
// and let the matrix cores run without vector work (and small batches get tiles that fill the
// chip, which the fused kernel's fixed 256 x 128 tile does not).  The GEMM moves
// both operands from global memory straight into LDS (buffer loads with the LDS modifier: no
// registers, no vector-ALU instructions) two K steps ahead through a ring of three LDS stages.
//
// Tile: 256 x 128 per workgroup, 8 wavefronts x (64 x 64 = 2 x 2 v_mfma_f32_32x32x16), or 128 x 128
// and 128 x 64 when the problem has too few large tiles to fill the chip; K in steps of 64.  LDS
// rows are 128 bytes, unpadded (the DMA writes 1 KB = 8 rows per wavefront instruction, lane l ->
// bytes 16 l ..), and 16-byte chunk c of row r is kept in slot
// c ^ ((r >> 1) & 7): 16 consecutive lanes of a fragment read then cover all 64 banks once.  The
// swizzle is applied on the global side: lane l of a DMA fetches chunk (l & 7) ^ ((r >> 1) & 7) of
// row r = 8 * block + (l >> 3), so every 128-byte row is still read as one full line.
#include "blocks.hpp"
#include "common.hpp"

#include <algorithm>
#include <type_traits>

#include <cstdlib>

namespace gq {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int DK = 64;
constexpr int ROWB = 128;  // bytes per LDS row

// a compile-time switch (std::true_type / std::false_type) or a run-time one (bool) behind one spelling
template <class F> __device__ __forceinline__ constexpr bool is_on(F f) {
    if constexpr (std::is_same_v<F, bool>) return f;
    else return F::value;
}

template <bool BF16> struct Op16;
template <> struct Op16<true> {
    typedef bf16x8 vec8;
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        bf2 v;
        v.x = (__bf16)a;
        v.y = (__bf16)b;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Op16<false> {
    typedef f16x8 vec8;
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 v;
        v.x = (_Float16)a;
        v.y = (_Float16)b;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

// K rounded up to the GEMM's step: both 16-bit images are written with this row length (zeros behind
// K), so any K that is a whole number of blocks goes through.
__host__ __device__ inline int64_t padded_k(int64_t K) { return (K + 63) / 64 * 64; }

// ---- pass 1: GGML blocks -> 16-bit [N, K] -------------------------------------------------------
// One thread per run of 16 weights (32 output bytes).  half = 0: image row = weight row.  half = 1 / 2:
// the matrix is the first / second of a gated pair, whose images interleave in chunks of 32 rows
// (image rows 64 c .. 64 c + 31 = rows 32 c .. of the first matrix, the next 32 = the same rows of
// the second), so that a wavefront's 64-column tile holds both projections of 32 outputs.
// The image's rows hold runs_per_row runs, of which the first `runs` come from W and the rest (padding
// of K to the GEMM's step of 64) are zero.
template <int T, bool BF16>
__device__ __forceinline__ void dequant16bit_body(const uint8_t *__restrict__ W, uint16_t *__restrict__ out, uint32_t runs_per_row,
                                                  uint32_t total_runs, int64_t row_bytes, int half, uint32_t runs, uint32_t block) {
    // The 16-byte halves of the runs meet in LDS so that consecutive lanes store consecutive 16 bytes
    // (whole cache lines per store instruction; a lane storing its own 32 bytes in two instructions
    // half-fills twice as many).  An image holds at most 2^27 runs: 32-bit index arithmetic.
    __shared__ uint4 halves[512];
    const uint32_t tid = threadIdx.x, g0 = block * 256u, g = g0 + tid;
    if (g < total_runs) {
        const uint32_t row = g / runs_per_row, run = g % runs_per_row;
        float w[16];
        if (run < runs) {
            dequant16<T>(W + (int64_t)row * row_bytes, run, w);
        } else {
#pragma unroll
            for (int i = 0; i < 16; i++) w[i] = 0.f;
        }
        halves[2 * tid] = make_uint4(Op16<BF16>::pack(w[0], w[1]), Op16<BF16>::pack(w[2], w[3]), Op16<BF16>::pack(w[4], w[5]),
                                     Op16<BF16>::pack(w[6], w[7]));
        halves[2 * tid + 1] = make_uint4(Op16<BF16>::pack(w[8], w[9]), Op16<BF16>::pack(w[10], w[11]), Op16<BF16>::pack(w[12], w[13]),
                                         Op16<BF16>::pack(w[14], w[15]));
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const uint32_t c = tid + 256u * p, gg = g0 + (c >> 1);
        if (gg >= total_runs) continue;
        const uint32_t row = gg / runs_per_row, run = gg % runs_per_row;
        const int64_t out_row = half == 0 ? (int64_t)row : (int64_t)(row >> 5) * 64 + (half - 1) * 32 + (row & 31);
        *reinterpret_cast<uint4 *>(out + (out_row * runs_per_row + run) * 16 + (c & 1u) * 8u) = halves[c];
    }
}

template <int T, bool BF16>
__global__ __launch_bounds__(256) void dequant16bit_kernel(const uint8_t *__restrict__ W, uint16_t *__restrict__ out, uint32_t runs_per_row,
                                                          uint32_t total_runs, int64_t row_bytes, int half, uint32_t runs) {
    dequant16bit_body<T, BF16>(W, out, runs_per_row, total_runs, row_bytes, half, runs, blockIdx.x);
}

// fp32 activations -> fp16 [M, K], one workgroup per row: the row is scaled by a power of two
// (pow2_scale) so that neither large nor tiny inputs leave fp16's range; rowscale[m] receives the
// inverse, which the GEMM's epilogue applies.  (The row is read twice, the second time from cache.)
__global__ __launch_bounds__(256) void x_to_f16_kernel(const float *__restrict__ X, int K, uint16_t *__restrict__ out, float *__restrict__ rowscale) {
    __shared__ float part[4];
    const float4 *x = reinterpret_cast<const float4 *>(X + (int64_t)blockIdx.x * K);
    const int k8 = K / 8, kp8 = (int)(padded_k(K) / 8);
    float am = 0.f;
    for (int g = threadIdx.x; g < k8; g += 256) am = fmaxf(am, amax8(x[2 * g], x[2 * g + 1]));
    am = wave_max(am);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = am;
    __syncthreads();
    float sc, inv;
    pow2_scale(fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3])), sc, inv);
    if (threadIdx.x == 0) rowscale[blockIdx.x] = inv;
    uint4 *o = reinterpret_cast<uint4 *>(out + (int64_t)blockIdx.x * (kp8 * 8));
    for (int g = threadIdx.x; g < kp8; g += 256) {
        if (g >= k8) { o[g] = make_uint4(0u, 0u, 0u, 0u); continue; }
        const float4 a = x[2 * g], b = x[2 * g + 1];
        o[g] = make_uint4(Op16<false>::pack(a.x * sc, a.y * sc), Op16<false>::pack(a.z * sc, a.w * sc), Op16<false>::pack(b.x * sc, b.y * sc),
                          Op16<false>::pack(b.z * sc, b.w * sc));
    }
}

// The same pass with an RMS normalisation in front: fp16(x / sqrt(mean(x^2) + eps) * (gain + offset)),
// one workgroup per activation row (the row is read twice, the second time from cache).  K % 8 == 0.
__global__ __launch_bounds__(256) void x_rmsnorm_to_f16_kernel(const float *__restrict__ X, const float *__restrict__ gain, float gain_offset,
                                                               float eps, int K, uint16_t *__restrict__ out, float *__restrict__ rowscale) {
    __shared__ float part[4];
    const float4 *x = reinterpret_cast<const float4 *>(X + (int64_t)blockIdx.x * K);
    const int k8 = K / 8, kp8 = (int)(padded_k(K) / 8);
    float ss = 0.f;
    for (int g = threadIdx.x; g < k8; g += 256) {
        const float4 a = x[2 * g], b = x[2 * g + 1];
        ss += (a.x * a.x + a.y * a.y) + (a.z * a.z + a.w * a.w) + (b.x * b.x + b.y * b.y) + (b.z * b.z + b.w * b.w);
    }
    for (int m = 1; m < 64; m <<= 1) ss += __shfl_xor(ss, m);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float r = sqrtf(((part[0] + part[1]) + (part[2] + part[3])) / (float)K + eps);
    if (threadIdx.x == 0) rowscale[blockIdx.x] = 1.f;  // normalised rows are O(gain): no scaling
    uint4 *o = reinterpret_cast<uint4 *>(out + (int64_t)blockIdx.x * (kp8 * 8));
    for (int g = threadIdx.x; g < kp8; g += 256) {
        if (g >= k8) { o[g] = make_uint4(0u, 0u, 0u, 0u); continue; }
        float4 a = x[2 * g], b = x[2 * g + 1];
        a.x /= r; a.y /= r; a.z /= r; a.w /= r; b.x /= r; b.y /= r; b.z /= r; b.w /= r;
        if (gain) {
            const float4 ga = reinterpret_cast<const float4 *>(gain)[2 * g], gb = reinterpret_cast<const float4 *>(gain)[2 * g + 1];
            a.x *= ga.x + gain_offset; a.y *= ga.y + gain_offset; a.z *= ga.z + gain_offset; a.w *= ga.w + gain_offset;
            b.x *= gb.x + gain_offset; b.y *= gb.y + gain_offset; b.z *= gb.z + gain_offset; b.w *= gb.w + gain_offset;
        }
        o[g] = make_uint4(Op16<false>::pack(a.x, a.y), Op16<false>::pack(a.z, a.w), Op16<false>::pack(b.x, b.y), Op16<false>::pack(b.z, b.w));
    }
}

// Both activation passes for rows of at most 2048 IT values: the row stays in registers between the reduction and
// the conversion, so it is read once.  NORM: the RMS normalisation variant.
template <int IT, bool NORM>
__device__ __forceinline__ void x_row_to_f16_body(const float *__restrict__ X, const float *__restrict__ gain, float gain_offset, float eps,
                                                  int K, uint16_t *__restrict__ out, float *__restrict__ rowscale, uint32_t row) {
    __shared__ float part[4];
    const float4 *x = reinterpret_cast<const float4 *>(X + (int64_t)row * K);
    const int k8 = K / 8, kp8 = (int)(padded_k(K) / 8);
    float4 a[IT], b[IT];
#pragma unroll
    for (int i = 0; i < IT; i++) {  // (groups past the row re-read its last one: no branch around the loads)
        const int g = min((int)threadIdx.x + 256 * i, k8 - 1);
        a[i] = x[2 * g];
        b[i] = x[2 * g + 1];
    }
    float red = 0.f;
#pragma unroll
    for (int i = 0; i < IT; i++) {
        if ((int)threadIdx.x + 256 * i >= k8) continue;
        if constexpr (NORM)
            red += (a[i].x * a[i].x + a[i].y * a[i].y) + (a[i].z * a[i].z + a[i].w * a[i].w) + (b[i].x * b[i].x + b[i].y * b[i].y) +
                   (b[i].z * b[i].z + b[i].w * b[i].w);
        else
            red = fmaxf(red, amax8(a[i], b[i]));
    }
    if constexpr (NORM) {
        for (int m = 1; m < 64; m <<= 1) red += __shfl_xor(red, m);
    } else {
        red = wave_max(red);
    }
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = red;
    __syncthreads();
    float sc = 1.f, r = 1.f;
    if constexpr (NORM) {
        r = sqrtf(((part[0] + part[1]) + (part[2] + part[3])) / (float)K + eps);
        if (threadIdx.x == 0) rowscale[row] = 1.f;  // normalised rows are O(gain): no scaling
    } else {
        float inv;
        pow2_scale(fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3])), sc, inv);
        if (threadIdx.x == 0) rowscale[row] = inv;
    }
    uint4 *o = reinterpret_cast<uint4 *>(out + (int64_t)row * (kp8 * 8));
#pragma unroll
    for (int i = 0; i < IT; i++) {
        const int g = (int)threadIdx.x + 256 * i;
        if (g >= kp8) continue;
        if (g >= k8) { o[g] = make_uint4(0u, 0u, 0u, 0u); continue; }
        float4 p = a[i], q = b[i];
        if constexpr (NORM) {
            p.x /= r; p.y /= r; p.z /= r; p.w /= r; q.x /= r; q.y /= r; q.z /= r; q.w /= r;
            if (gain) {
                const float4 ga = reinterpret_cast<const float4 *>(gain)[2 * g], gb = reinterpret_cast<const float4 *>(gain)[2 * g + 1];
                p.x *= ga.x + gain_offset; p.y *= ga.y + gain_offset; p.z *= ga.z + gain_offset; p.w *= ga.w + gain_offset;
                q.x *= gb.x + gain_offset; q.y *= gb.y + gain_offset; q.z *= gb.z + gain_offset; q.w *= gb.w + gain_offset;
            }
        } else {
            p.x *= sc; p.y *= sc; p.z *= sc; p.w *= sc; q.x *= sc; q.y *= sc; q.z *= sc; q.w *= sc;
        }
        o[g] = make_uint4(Op16<false>::pack(p.x, p.y), Op16<false>::pack(p.z, p.w), Op16<false>::pack(q.x, q.y), Op16<false>::pack(q.z, q.w));
    }
}

template <int IT, bool NORM>
__global__ __launch_bounds__(256) void x_row_to_f16_kernel(const float *__restrict__ X, const float *__restrict__ gain, float gain_offset, float eps,
                                                           int K, uint16_t *__restrict__ out, float *__restrict__ rowscale) {
    x_row_to_f16_body<IT, NORM>(X, gain, gain_offset, eps, K, out, rowscale, blockIdx.x);
}

// x -> fp16 rows (+ row scales), with the normalisation when norm is given
int launch_x_to_f16(const float *x, int64_t M, int64_t K, const RmsNorm *norm, uint16_t *xh, float *rowscale, hipStream_t s) {
    const dim3 grid((unsigned)M), block(256);
    const float *gain = norm ? norm->gain : nullptr;
    const float off = norm ? norm->gain_offset : 0.f, eps = norm ? norm->eps : 0.f;
    const int64_t kp = padded_k(K);
    if (kp <= 4096)
        return norm ? launch(x_row_to_f16_kernel<2, true>, grid, block, 0, s, x, gain, off, eps, (int)K, xh, rowscale)
                    : launch(x_row_to_f16_kernel<2, false>, grid, block, 0, s, x, gain, off, eps, (int)K, xh, rowscale);
    if (kp <= 8192)
        return norm ? launch(x_row_to_f16_kernel<4, true>, grid, block, 0, s, x, gain, off, eps, (int)K, xh, rowscale)
                    : launch(x_row_to_f16_kernel<4, false>, grid, block, 0, s, x, gain, off, eps, (int)K, xh, rowscale);
    if (kp <= 16384)
        return norm ? launch(x_row_to_f16_kernel<8, true>, grid, block, 0, s, x, gain, off, eps, (int)K, xh, rowscale)
                    : launch(x_row_to_f16_kernel<8, false>, grid, block, 0, s, x, gain, off, eps, (int)K, xh, rowscale);
    return norm ? launch(x_rmsnorm_to_f16_kernel, grid, block, 0, s, x, gain, off, eps, (int)K, xh, rowscale)
                : launch(x_to_f16_kernel, grid, block, 0, s, x, (int)K, xh, rowscale);
}

// ---- pass 2: 16-bit GEMM with global -> LDS DMA --------------------------------------------------
// One 16-byte-per-lane buffer load whose data goes to LDS at lds_addr + 16 * lane.  The compiler
// does not see that the instruction writes LDS or that it is counted by vmcnt: the kernel orders
// these loads against its LDS reads with explicit waits and barriers.  (The s_nop is the wait
// state the hardware wants between a write of M0 and an LDS DMA; the assembler does not add it
// inside inline assembly.)
__device__ __forceinline__ void dma16(uint32_t lds_addr, i32x4 rsrc, uint32_t voff, uint32_t soff) {
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);  // both are uniform by construction
    soff = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}

__device__ __forceinline__ i32x4 make_rsrc(const void *base, uint64_t bytes) {
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    i32x4 r;
    r.x = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    r.y = __builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));  // stride 0: raw buffer, byte offsets
    r.z = __builtin_amdgcn_readfirstlane((int)(uint32_t)(bytes > 0xFFFFFFFFull ? 0xFFFFFFFFull : bytes));
    r.w = 0x00020000;  // 32-bit data format, no swizzle
    return r;
}

// X [M, K] and Wh [N, K] 16-bit, K % 64 == 0, both 16-byte aligned.  The workgroup tile is
// (128 TM) x (64 TN): 4 x 2 wavefronts of (32 TM) x (32 TN) each.  TM = TN = 2 is the tile for
// large problems; the smaller ones keep the chip full when M x N yields too few big tiles.
template <int TM, int TN> struct DmaTile {
    static constexpr int DM = 128 * TM, DN = 64 * TN;
    static constexpr int XI = 2 * TM, WI = TN;                 // DMAs per wavefront and step: X, W
    static constexpr int kStageBytes = (DM + DN) * ROWB;
    // Three stages: deeper rings for the small tiles (4 and 6 stages fit) measured slightly slower,
    // because they leave room for one workgroup per CU instead of two.  (Also measured: the 256 x 128
    // tile on four wavefronts of 128 x 64, which reads a quarter less from LDS per MFMA but leaves a
    // SIMD a single wavefront: 112 .. 120 us against 81 .. 89 us at 2048 rows.)
    static constexpr int NS = 3;
    static constexpr int kLdsBytes = NS * kStageBytes;
};

// GATED (TN == 2): Wh is the interleaved image of a gated pair (N counts its rows); column block j = 0
// of a wavefront's tile is the first projection, j = 1 the second, of the same 32 outputs, and the
// result is act(first + bias) * (second + bias2) in a [M, n_out] matrix.
// SEGS: the image is several matrices one after the other (N counts all their rows) and the columns of the result go to
// one output matrix per segment: columns n0[i] .. n0[i + 1] - 1 to y[i] (row length n0[i + 1] - n0[i]) with bias[i]; the
// boundaries are multiples of 32, so a wavefront's block of 32 columns lies in one segment.
// gridDim.z > 1 (not GATED): K is split into that many slices of whole steps; slice z contracts its steps only and writes
// its [M, N] sums behind those of the slices before it (Y + z M N), for gemm_slices_reduce_kernel to add up and finish.
struct GemmSegs {
    float *y[4];
    const float *bias[4];
    int n0[5];
    int count;
};

template <bool BF16, int TM, int TN, bool GATED = false, bool SEGS = false>
__global__ __launch_bounds__(512) void gemm_dma_kernel(const uint16_t *X, const uint16_t *Wh, const float *__restrict__ bias,
                                                       float *Y, int M, int K, int N, int act, const float *__restrict__ bias2, int n_out,
                                                       const float *residual, const float *__restrict__ rowscale, GemmSegs segs) {
    typedef Op16<BF16> Op;
    typedef DmaTile<TM, TN> G;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bm = blockIdx.y * G::DM, bn = blockIdx.x * G::DN;
    const int wm = (wave >> 1) * (32 * TM), wn = (wave & 1) * (32 * TN);
    const int nk_all = K / DK, nk_slice = (nk_all + (int)gridDim.z - 1) / (int)gridDim.z;
    const int k0 = (int)blockIdx.z * nk_slice;       // (the host gives every slice at least one step)
    const int nk = min(nk_slice, nk_all - k0);

    // ---- DMA roles: per step a wavefront moves XI row blocks (8 rows each) of X and WI of W
    const i32x4 xrsrc = make_rsrc(X + (int64_t)bm * K, (uint64_t)(M - bm) * (uint64_t)K * 2);
    const i32x4 wrsrc = make_rsrc(Wh + (int64_t)bn * K, (uint64_t)(N - bn) * (uint64_t)K * 2);
    uint32_t xvoff[G::XI], wvoff[G::WI];
#pragma unroll
    for (int j = 0; j < G::XI; j++) {
        const int row = 8 * (G::XI * wave + j) + (lane >> 3);
        const int c = (lane & 7) ^ ((row >> 1) & 7);
        xvoff[j] = (uint32_t)min(row, M - 1 - bm) * (uint32_t)(K * 2) + (uint32_t)c * 16u;
    }
#pragma unroll
    for (int j = 0; j < G::WI; j++) {
        const int row = 8 * (G::WI * wave + j) + (lane >> 3);
        const int c = (lane & 7) ^ ((row >> 1) & 7);
        wvoff[j] = (uint32_t)min(row, N - 1 - bn) * (uint32_t)(K * 2) + (uint32_t)c * 16u;
    }
    const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>(lds);
    const uint32_t xdst = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)(G::XI * wave) * 1024u);
    const uint32_t wdst = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)(G::DM * ROWB) + (uint32_t)(G::WI * wave) * 1024u);
    auto issue = [&](int kt, int stage) __attribute__((always_inline)) {  // steps past the end re-read the last one (the data is never used)
        const uint32_t soff = (uint32_t)(k0 + min(kt, nk - 1)) * (uint32_t)(DK * 2);
        const uint32_t sb = (uint32_t)stage * (uint32_t)G::kStageBytes;
#pragma unroll
        for (int j = 0; j < G::XI; j++) dma16(xdst + sb + (uint32_t)j * 1024u, xrsrc, xvoff[j], soff);
#pragma unroll
        for (int j = 0; j < G::WI; j++) dma16(wdst + sb + (uint32_t)j * 1024u, wrsrc, wvoff[j], soff);
    };

    // ---- fragment addresses: row (w? + 32 t + lane % 32), chunk 2 kk + lane / 32, swizzled
    uint32_t aoff[4], boff[4];
    {
        const int l = lane & 31, sw = (l >> 1) & 7, hi = lane >> 5;  // wm, wn, 32 t are multiples of 16
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            const uint32_t slot = (uint32_t)((2 * kk + hi) ^ sw);
            aoff[kk] = (uint32_t)(wm + l) * ROWB + slot * 16u;
            boff[kk] = (uint32_t)(G::DM * ROWB) + (uint32_t)(wn + l) * ROWB + slot * 16u;
        }
    }

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    typename Op::vec8 fa[2][TM], fb[2][TN];  // [set][tile]
    auto frags = [&](int stage, int kk) __attribute__((always_inline)) {
        const uint8_t *base = lds + stage * G::kStageBytes;
        const int set = kk & 1;
#pragma unroll
        for (int t = 0; t < TM; t++) fa[set][t] = *reinterpret_cast<const typename Op::vec8 *>(base + aoff[kk] + t * 32 * ROWB);
#pragma unroll
        for (int t = 0; t < TN; t++) fb[set][t] = *reinterpret_cast<const typename Op::vec8 *>(base + boff[kk] + t * 32 * ROWB);
    };
    auto mfma_group = [&](int set) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) acc[i][j] = Op::mfma(fa[set][i], fb[set][j], acc[i][j]);
    };
    // Waits until this wavefront's DMAs of the next step have landed (those of the NS - 2 steps after
    // it may stay in flight) and its own LDS reads are done, then meets the other wavefronts.
    auto publish = [&]() __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((G::NS - 2) * (G::XI + G::WI)) : "memory");
    };

#pragma unroll
    for (int p = 0; p < G::NS - 1; p++) issue(p, p);
    publish();
    // Step kt computes out of stage kt % NS while the DMAs of step kt + NS - 1 fill the stage that
    // every wavefront finished reading before the barrier that ended step kt - 1.  The MFMA groups
    // are skewed by one against the barriers (group 3 of a step issues after the barrier, behind
    // the first fragment reads of the next step).
    auto step = [&](int kt, int stage, bool first) __attribute__((always_inline)) {
        issue(kt + G::NS - 1, (stage + G::NS - 1) % G::NS);
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            frags(stage, kk);
            if (kk > 0 || !first) mfma_group((kk + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        publish();
    };
    step(0, 0, true);
    int kt = 1;
    for (; kt + G::NS - 1 < nk; kt += G::NS) {  // stages 1, 2, .., NS - 1, 0: compile-time LDS offsets
#pragma unroll
        for (int p = 0; p < G::NS; p++) step(kt + p, (1 + p) % G::NS, false);
    }
#pragma unroll
    for (int p = 0; p < G::NS - 1; p++)
        if (kt < nk) { step(kt, 1 + p, false); kt++; }
    mfma_group(1);  // group 3 of the last step
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the re-read DMAs of the last steps

    // ---- epilogue: acc[i][j][r] is Y[m, n] with n = lane % 32, m = 8*(r/4) + 4*(lane/32) + r%4
    // Per element: an add (or a multiply-add with the row's scale), the activation, a store; the address is a per-lane base
    // plus an offset that is the same for the whole wavefront, and everything that does not depend on the element - which
    // activation, row scales or not, residual or not, whether the tile reaches over the edge of the matrix - is decided
    // once, outside the 64 stores.  (Written as one loop with those tests inside, the compiler spent some twenty vector-ALU
    // instructions per element: C3 through the two passes took 83.3 us against 75.9, fp32 prefill 98.3 against 87.3.)
    const int m0 = bm + wm + 4 * (lane >> 5);
    if constexpr (GATED) {
        static_assert(TN == 2, "a gated tile pairs two 32-column blocks");
        // (the image of a gated pair may have more rows than 2 n_out: the bound is on the output columns)
        const int n = ((bn + wn) >> 1) + (lane & 31);
        if (n >= n_out) return;
        const float bg = bias ? bias[n] : 0.f, bu = bias2 ? bias2[n] : 0.f;
        const int64_t at0 = (int64_t)m0 * n_out + n;
        auto store_all = [&](auto bounded, auto scaled, auto with_residual, auto activate) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < TM; i++) {
                const int rows_left = decltype(bounded)::value ? M - (bm + wm + i * 32) : 32;  // (see the plain form below)
                if (rows_left <= 0) continue;
                auto store16 = [&](auto checked) __attribute__((always_inline)) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int dm = i * 32 + 8 * (r >> 2) + (r & 3);
                        if constexpr (decltype(checked)::value) { if (m0 + dm >= M) continue; }
                        float rs = 1.f;
                        if (is_on(scaled)) rs = rowscale[m0 + dm];
                        float v = activate(fmaf(acc[i][0][r], rs, bg)) * fmaf(acc[i][1][r], rs, bu);
                        if (is_on(with_residual)) v += residual[at0 + (int64_t)dm * n_out];
                        Y[at0 + (int64_t)dm * n_out] = v;
                    }
                };
                if (rows_left >= 32) store16(std::false_type());
                else store16(std::true_type());
            }
        };
        // (SiLU, the activation of the feed-forward blocks this form exists for, gets the compile-time switches; the
        // others take row scales and residual as run-time tests, uniform over the wavefront: a quarter of the code)
        auto by_edge = [&](auto bounded) __attribute__((always_inline)) {
            auto silu = [](float v) { return v / (1.0f + __expf(-v)); };
            if (act != kActSilu) store_all(bounded, rowscale != nullptr, residual != nullptr, [act](float v) { return apply_act(act, v); });
            else if (rowscale && residual) store_all(bounded, std::true_type(), std::true_type(), silu);
            else if (rowscale) store_all(bounded, std::true_type(), std::false_type(), silu);
            else if (residual) store_all(bounded, std::false_type(), std::true_type(), silu);
            else store_all(bounded, std::false_type(), std::false_type(), silu);
        };
        if (bm + G::DM <= M) by_edge(std::false_type());
        else by_edge(std::true_type());
        return;
    }
    float *const Yall = Y + (int64_t)blockIdx.z * (int64_t)M * (int64_t)N;
    const float *const bias_all = bias;
    const int Nall = N;
    auto store_all = [&](auto bounded, auto scaled, auto with_residual, auto activate) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            int n = bn + wn + j * 32 + (lane & 31);
            if constexpr (decltype(bounded)::value) { if (n >= N) continue; }
            float *Y = Yall;               // (shadow the kernel's arguments: a segment brings its own output, row length and bias)
            const float *bias = bias_all;
            int N = Nall;
            if constexpr (SEGS) {
                int sg = 0;
#pragma unroll
                for (int q = 1; q < 4; q++)
                    if (q < segs.count && n >= segs.n0[q]) sg = q;
                Y = segs.y[sg];
                bias = segs.bias[sg];
                N = segs.n0[sg + 1] - segs.n0[sg];
                n -= segs.n0[sg];
            }
            const float bv = bias ? bias[n] : 0.f;
            const int64_t at0 = (int64_t)m0 * N + n;
#pragma unroll
            for (int i = 0; i < TM; i++) {
                // a block of 32 rows is inside the matrix as a whole, outside as a whole, or (one block per tile column at most) cut by its edge
                const int rows_left = decltype(bounded)::value ? M - (bm + wm + i * 32) : 32;
                if (rows_left <= 0) continue;
                auto store16 = [&](auto checked) __attribute__((always_inline)) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int dm = i * 32 + 8 * (r >> 2) + (r & 3);
                        if constexpr (decltype(checked)::value) { if (m0 + dm >= M) continue; }
                        float v = acc[i][j][r];
                        if (is_on(scaled)) v = fmaf(v, rowscale[m0 + dm], bv);
                        else v += bv;
                        v = activate(v);
                        // (a residual may be Y itself: one thread reads and writes an element)
                        if (is_on(with_residual)) v += residual[at0 + (int64_t)dm * N];
                        Y[at0 + (int64_t)dm * N] = v;
                    }
                };
                if (rows_left >= 32) store16(std::false_type());
                else store16(std::true_type());
            }
        }
    };
    // (no activation - the projections of a decoder - gets the compile-time switches; with an activation, row scales and
    // residual are run-time tests, uniform over the wavefront: a quarter of the code)
    auto by_edge = [&](auto bounded) __attribute__((always_inline)) {
        auto none = [](float v) { return v; };
        if (act != kActNone) store_all(bounded, rowscale != nullptr, residual != nullptr, [act](float v) { return apply_act(act, v); });
        else if (rowscale && residual) store_all(bounded, std::true_type(), std::true_type(), none);
        else if (rowscale) store_all(bounded, std::true_type(), std::false_type(), none);
        else if (residual) store_all(bounded, std::false_type(), std::true_type(), none);
        else store_all(bounded, std::false_type(), std::false_type(), none);
    };
    if (bm + G::DM <= M && bn + G::DN <= N) by_edge(std::false_type());
    else by_edge(std::true_type());
}

// The sums of a GEMM whose K was split into slices: partial[z][m][n] added in slice order, then what the GEMM's own
// epilogue does for an unsplit one - row scale, bias, activation, residual (which may be Y itself), and with segments
// each column to its matrix's output.  N and the segment boundaries are multiples of 4: a thread owns four columns of a row.
__global__ __launch_bounds__(256) void gemm_slices_reduce_kernel(const float *__restrict__ partial, int slices, int M, int N,
                                                                 const float *__restrict__ rowscale, const float *__restrict__ bias, int act,
                                                                 const float *residual, float *Y, GemmSegs segs, int use_segs) {
    const int64_t MN = (int64_t)M * N;
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= MN) return;
    const int m = MN <= (int64_t)INT32_MAX ? (int)((uint32_t)i / (uint32_t)N) : (int)(i / N);
    int n = (int)(i - (int64_t)m * N);
    float4 v[8];  // (eight slices at most: all loads issued before the first sum)
#pragma unroll
    for (int z = 0; z < 8; z++) v[z] = *reinterpret_cast<const float4 *>(partial + (int64_t)min(z, slices - 1) * MN + i);
    float4 t = v[0];
#pragma unroll
    for (int z = 1; z < 8; z++)
        if (z < slices) { t.x += v[z].x; t.y += v[z].y; t.z += v[z].z; t.w += v[z].w; }
    int64_t at = i;
    if (use_segs) {
        int sg = 0;
#pragma unroll
        for (int q = 1; q < 4; q++)
            if (q < segs.count && n >= segs.n0[q]) sg = q;
        Y = segs.y[sg];
        bias = segs.bias[sg];
        n -= segs.n0[sg];
        at = (int64_t)m * (segs.n0[sg + 1] - segs.n0[sg]) + n;
    }
    if (rowscale) { const float rs = rowscale[m]; t.x *= rs; t.y *= rs; t.z *= rs; t.w *= rs; }
    if (bias) { const float4 b = *reinterpret_cast<const float4 *>(bias + n); t.x += b.x; t.y += b.y; t.z += b.z; t.w += b.w; }
    t = make_float4(apply_act(act, t.x), apply_act(act, t.y), apply_act(act, t.z), apply_act(act, t.w));
    if (residual) { const float4 r = *reinterpret_cast<const float4 *>(residual + at); t.x += r.x; t.y += r.y; t.z += r.z; t.w += r.w; }
    *reinterpret_cast<float4 *>(Y + at) = t;
}

template <int T, bool BF16>
int launch_dequant16bit(const uint8_t *W, int64_t N, int64_t K, uint16_t *out, hipStream_t s, int half) {
    const int64_t runs = K / 16, runs_per_row = padded_k(K) / 16, total = N * runs_per_row;
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    if (total > ((int64_t)1 << 27)) return fail(GQ_ERR_INVALID, "gemm: a 16-bit image of %lld x %lld values is too large", (long long)N, (long long)K);
    return launch(dequant16bit_kernel<T, BF16>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, W, out, (uint32_t)runs_per_row, (uint32_t)total,
                  row_bytes, half, (uint32_t)runs);
}

template <bool BF16>
int launch_dequant16bit_type(int type, const uint8_t *W, int64_t N, int64_t K, uint16_t *out, hipStream_t s, int half = 0) {
    switch (type) {
    case kQ4_0: return launch_dequant16bit<kQ4_0, BF16>(W, N, K, out, s, half);
    case kQ8_0: return launch_dequant16bit<kQ8_0, BF16>(W, N, K, out, s, half);
    case kIQ4_NL: return launch_dequant16bit<kIQ4_NL, BF16>(W, N, K, out, s, half);
    case kQ4_K: return launch_dequant16bit<kQ4_K, BF16>(W, N, K, out, s, half);
    case kQ6_K: return launch_dequant16bit<kQ6_K, BF16>(W, N, K, out, s, half);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "qdense: ggml type %d is not implemented", type);
    }
}

// Both pre-passes of the fp32-activation route in ONE launch (they do not depend on each other): the first M workgroups
// convert an activation row each (x_row_to_f16_body), the others 256 runs of weights each (dequant16bit_body), of W and -
// for a gated pair, whose images interleave - of W2.  Rows of up to 16384 values (longer ones keep their own two-read kernel).
// The matrices of one pre-pass: matrix i is W[i] with rows[i] rows, written from image row row0[i] on with the interleaving
// `half[i]` of dequant16bit_body (a gated pair: both matrices at row 0 with halves 1 and 2; a set: halves 0, one after the other).
struct PrepMatrices {
    const uint8_t *W[4];
    uint32_t rows[4], row0[4], blocks_end[4];  // blocks_end[i]: workgroups of matrices 0 .. i
    int half[4], count;
};

template <int T, int IT, bool NORM>
__global__ __launch_bounds__(256) void prep_f32_kernel(const float *__restrict__ X, const float *__restrict__ gain, float gain_offset, float eps, int K,
                                                       uint16_t *__restrict__ xh, float *__restrict__ rowscale, uint32_t xblocks, PrepMatrices pm,
                                                       uint16_t *__restrict__ wh, uint32_t runs_per_row, int64_t row_bytes, uint32_t runs) {
    const uint32_t b = blockIdx.x;
    if (b < xblocks) {
        x_row_to_f16_body<IT, NORM>(X, gain, gain_offset, eps, K, xh, rowscale, b);
        return;
    }
    const uint32_t wb = b - xblocks;
    int i = 0;
#pragma unroll
    for (int q = 1; q < 4; q++)
        if (q < pm.count && wb >= pm.blocks_end[q - 1]) i = q;
    const uint32_t first = i ? pm.blocks_end[i - 1] : 0u;
    dequant16bit_body<T, false>(pm.W[i], wh + (size_t)pm.row0[i] * runs_per_row * 16, runs_per_row, pm.rows[i] * runs_per_row, row_bytes, pm.half[i], runs,
                                wb - first);
}

template <int T>
int launch_prep_f32_t(const float *x, int64_t M, int64_t K, const RmsNorm *norm, uint16_t *xh, float *rowscale, PrepMatrices pm, uint16_t *wh,
                      hipStream_t s) {
    const int64_t runs = K / 16, runs_per_row = padded_k(K) / 16;
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    int64_t wblocks = 0;
    for (int i = 0; i < pm.count; i++) {
        const int64_t total = (int64_t)pm.rows[i] * runs_per_row;
        if (total > ((int64_t)1 << 27)) return fail(GQ_ERR_INVALID, "gemm: a 16-bit image of %u x %lld values is too large", pm.rows[i], (long long)K);
        wblocks += (total + 255) / 256;
        if (wblocks > INT32_MAX) return fail(GQ_ERR_INVALID, "gemm: too many workgroups in the pre-pass");
        pm.blocks_end[i] = (uint32_t)wblocks;
    }
    const int64_t blocks = M + wblocks;
    if (blocks > INT32_MAX) return fail(GQ_ERR_INVALID, "gemm: too many workgroups in the pre-pass");
    const float *gain = norm ? norm->gain : nullptr;
    const float off = norm ? norm->gain_offset : 0.f, eps = norm ? norm->eps : 0.f;
    const dim3 grid((unsigned)blocks), block(256);
    auto go = [&](auto kernel) {
        return launch(kernel, grid, block, 0, s, x, gain, off, eps, (int)K, xh, rowscale, (uint32_t)M, pm, wh, (uint32_t)runs_per_row, row_bytes, (uint32_t)runs);
    };
    if (padded_k(K) <= 4096) return norm ? go(prep_f32_kernel<T, 2, true>) : go(prep_f32_kernel<T, 2, false>);
    if (padded_k(K) <= 8192) return norm ? go(prep_f32_kernel<T, 4, true>) : go(prep_f32_kernel<T, 4, false>);
    return norm ? go(prep_f32_kernel<T, 8, true>) : go(prep_f32_kernel<T, 8, false>);
}

// x -> fp16 rows and the matrices -> fp16 image: one launch for rows of up to 16384 values (64 per thread in registers; on its
// own the activation pass of 128 rows of 14336 values took 6 us, a workgroup per row with nothing beside it), else one per operand
int launch_prep_f32(int type, const float *x, int64_t M, int64_t K, const RmsNorm *norm, uint16_t *xh, float *rowscale, const PrepMatrices &pm,
                    uint16_t *wh, hipStream_t s) {
    if (padded_k(K) > 16384) {
        if (int rc = launch_x_to_f16(x, M, K, norm, xh, rowscale, s)) return rc;
        for (int i = 0; i < pm.count; i++)
            if (int rc = launch_dequant16bit_type<false>(type, pm.W[i], pm.rows[i], K, wh + (size_t)pm.row0[i] * padded_k(K), s, pm.half[i])) return rc;
        return GQ_OK;
    }
    switch (type) {
    case kQ4_0: return launch_prep_f32_t<kQ4_0>(x, M, K, norm, xh, rowscale, pm, wh, s);
    case kQ8_0: return launch_prep_f32_t<kQ8_0>(x, M, K, norm, xh, rowscale, pm, wh, s);
    case kIQ4_NL: return launch_prep_f32_t<kIQ4_NL>(x, M, K, norm, xh, rowscale, pm, wh, s);
    case kQ4_K: return launch_prep_f32_t<kQ4_K>(x, M, K, norm, xh, rowscale, pm, wh, s);
    case kQ6_K: return launch_prep_f32_t<kQ6_K>(x, M, K, norm, xh, rowscale, pm, wh, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "qdense: ggml type %d is not implemented", type);
    }
}

// one matrix, or the two of a gated pair
PrepMatrices prep_one_or_pair(const uint8_t *W, const uint8_t *W2, int64_t N) {
    PrepMatrices pm{};
    pm.count = W2 ? 2 : 1;
    pm.W[0] = W; pm.rows[0] = (uint32_t)N; pm.row0[0] = 0; pm.half[0] = W2 ? 1 : 0;
    pm.W[1] = W2; pm.rows[1] = (uint32_t)N; pm.row0[1] = 0; pm.half[1] = 2;
    return pm;
}

// N counts the rows of the weight image (for a gated pair: both halves, 64 per 32 outputs)
template <bool BF16, int TM, int TN, bool GATED = false, bool SEGS = false>
int launch_gemm16_tile(const uint16_t *x, int64_t M, int64_t K, const uint16_t *Wh, int64_t N, const float *bias, int act, float *y,
                       const float *bias2, int64_t n_out, const float *residual, const float *rowscale, hipStream_t s,
                       const GemmSegs *segs = nullptr, int slices = 1) {
    typedef DmaTile<TM, TN> G;
    static const bool lds_ok = [] {
        return hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_dma_kernel<BF16, TM, TN, GATED, SEGS>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, G::kLdsBytes) == hipSuccess;
    }();
    if (!lds_ok) return fail(GQ_ERR_HIP, "gemm: cannot reserve %d bytes of LDS", G::kLdsBytes);
    static_assert(!GATED || !SEGS, "a gated pair has one output");
    if (slices < 1 || (GATED && slices != 1) || (int64_t)(slices - 1) * ((K / DK + slices - 1) / slices) >= K / DK)
        return fail(GQ_ERR_INVALID, "gemm: %d slices of K = %lld", slices, (long long)K);
    const dim3 grid((unsigned)((N + G::DN - 1) / G::DN), (unsigned)((M + G::DM - 1) / G::DM), (unsigned)slices);
    return launch(gemm_dma_kernel<BF16, TM, TN, GATED, SEGS>, grid, dim3(512), (size_t)G::kLdsBytes, s, x, Wh, bias, y, (int)M, (int)K, (int)N, act,
                  bias2, (int)n_out, residual, rowscale, segs ? *segs : GemmSegs{});
}

// GOMLX_HIPQ_GEMM_TILE=0|1|2 forces the 256x128 / 128x128 / 128x64 tile (tuning runs only).
int tile_env() {
    static const int v = [] { const char *e = std::getenv("GOMLX_HIPQ_GEMM_TILE"); return e ? std::atoi(e) : -1; }();
    return v;
}

// Which tile: 0 = 256 x 128, 1 = 128 x 128 (one workgroup per CU each), 2 = 128 x 64 (two per CU).  The workgroups run in
// rounds of one per CU; a round of 128 x 128 tiles takes about 0.61 of a round of 256 x 128 tiles, and a last round that is
// only partly filled still costs a good half of a full one (the chip clocks higher and the memory system is less
// crowded, but every workgroup walks all of K).  Estimated that way, the choice matches the faster tile in 22 of 24
// measured cases (K = 4096 and 14336, N = 4096 and 14336, 640 .. 1536 rows) - e.g. 1280 rows on 4096 x 4096 are 160
// large tiles in one round (57 us) or 320 small ones in two (70 us), where a rule by tile count alone took the small ones.
int pick_tile(int64_t M, int64_t N) {
    const int64_t cus = device_cu_count();
    auto tiles = [&](int64_t dm, int64_t dn) { return ((M + dm - 1) / dm) * ((N + dn - 1) / dn); };
    if (tiles(128, 64) <= cus) return 2;  // small problems: as long as the smallest tiles run in one round they win (512 rows on 4096 x 4096: 35 against 38 us; 640 rows: 48 against 39)
    if (M <= 128) return 1;                       // (no half-empty 256-row tiles)
    auto rounds = [&](int64_t wgs, double empty_round) {
        const int64_t full = wgs / cus;
        const double frac = (double)(wgs % cus) / (double)cus;
        return (double)full + (frac > 0.0 ? empty_round + (1.0 - empty_round) * frac : 0.0);
    };
    const double t0 = rounds(tiles(256, 128), 0.6), t1 = 0.61 * rounds(tiles(128, 128), 0.5);
    return t0 <= t1 ? 0 : 1;
}

// Few rows on a matrix with few columns leave most of the chip without a workgroup, each of the few walking all of K
// (128 rows on 14336 -> 4096: 64 tiles of 128 x 64 on 256 CUs).  Then K is split into slices, as many as fill the chip
// with at least 16 steps (1024 values) each, eight at most; the slices' sums go to `partial` ([slices][M][N] fp32) and a
// small kernel adds them up and finishes them.  GOMLX_HIPQ_GEMM_K_SLICES=n forces n where it applies (1: never split).
int k_slices_env() {
    static const int v = [] { const char *e = std::getenv("GOMLX_HIPQ_GEMM_K_SLICES"); return e ? std::atoi(e) : 0; }();
    return v;
}
int gemm_k_slices(int64_t M, int64_t K, int64_t N) {
    if (N % 4 != 0) return 1;
    const int64_t steps = K / DK, tiles = ((M + 127) / 128) * ((N + 63) / 64);
    int64_t ns = std::min<int64_t>(std::min<int64_t>(device_cu_count() / tiles, steps / 16), 8);
    if (k_slices_env() > 0) ns = std::min<int64_t>(std::min<int64_t>(k_slices_env(), steps), 8);
    while (ns > 1 && (ns - 1) * ((steps + ns - 1) / ns) >= steps) ns--;  // no empty slice
    return ns < 2 ? 1 : (int)ns;
}
size_t gemm_partial_bytes(int64_t M, int64_t K, int64_t N) {
    const int ns = gemm_k_slices(M, K, N);
    return ns > 1 ? (size_t)ns * (size_t)M * (size_t)N * sizeof(float) : 0;
}
template <class... P> bool aligned16(P... p) { return (((reinterpret_cast<uintptr_t>(p)) | ...) & 15) == 0; }  // (the reduction's float4 accesses)
int launch_slices_reduce(const float *partial, int slices, int64_t M, int64_t N, const float *rowscale, const float *bias, int act,
                         const float *residual, float *y, const GemmSegs *segs, hipStream_t s) {
    const int64_t quads = M * N / 4;
    return launch(gemm_slices_reduce_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, partial, slices, (int)M, (int)N, rowscale, bias, act,
                  residual, y, segs ? *segs : GemmSegs{}, segs ? 1 : 0);
}

// partial: room for gemm_partial_bytes(M, K, N), or null (then K is never split)
template <bool BF16>
int launch_gemm16(const uint16_t *x, int64_t M, int64_t K, const uint16_t *Wh, int64_t N, const float *bias, int act, float *y, hipStream_t s,
                  const float *residual = nullptr, const float *rowscale = nullptr, float *partial = nullptr) {
    if (const int ns = partial && aligned16(bias, residual, y) ? gemm_k_slices(M, K, N) : 1; ns > 1) {
        if (int rc = launch_gemm16_tile<BF16, 1, 1>(x, M, K, Wh, N, nullptr, kActNone, partial, nullptr, N, nullptr, nullptr, s, nullptr, ns)) return rc;
        return launch_slices_reduce(partial, ns, M, N, rowscale, bias, act, residual, y, nullptr, s);
    }
    int choice = pick_tile(M, N);
    if (tile_env() >= 0 && tile_env() <= 2) choice = tile_env();
    switch (choice) {
    case 0: return launch_gemm16_tile<BF16, 2, 2>(x, M, K, Wh, N, bias, act, y, nullptr, N, residual, rowscale, s);
    case 1: return launch_gemm16_tile<BF16, 1, 2>(x, M, K, Wh, N, bias, act, y, nullptr, N, residual, rowscale, s);
    default: return launch_gemm16_tile<BF16, 1, 1>(x, M, K, Wh, N, bias, act, y, nullptr, N, residual, rowscale, s);
    }
}

// Several matrices' images one after the other, one GEMM, each segment's columns to its own output (fp16 operands).
int launch_gemm16_set(const uint16_t *x, int64_t M, int64_t K, const uint16_t *Wh, const GemmSegs &segs, int act, const float *rowscale, hipStream_t s,
                      float *partial) {
    const int64_t N = segs.n0[segs.count];
    bool aligned = true;
    for (int i = 0; i < segs.count; i++) aligned = aligned && aligned16(segs.bias[i], segs.y[i]);
    if (const int ns = partial && aligned ? gemm_k_slices(M, K, N) : 1; ns > 1) {
        if (int rc = launch_gemm16_tile<false, 1, 1>(x, M, K, Wh, N, nullptr, kActNone, partial, nullptr, N, nullptr, nullptr, s, nullptr, ns)) return rc;
        return launch_slices_reduce(partial, ns, M, N, rowscale, nullptr, act, nullptr, nullptr, &segs, s);
    }
    int choice = pick_tile(M, N);
    if (tile_env() >= 0 && tile_env() <= 2) choice = tile_env();
    switch (choice) {
    case 0: return launch_gemm16_tile<false, 2, 2, false, true>(x, M, K, Wh, N, nullptr, act, nullptr, nullptr, N, nullptr, rowscale, s, &segs);
    case 1: return launch_gemm16_tile<false, 1, 2, false, true>(x, M, K, Wh, N, nullptr, act, nullptr, nullptr, N, nullptr, rowscale, s, &segs);
    default: return launch_gemm16_tile<false, 1, 1, false, true>(x, M, K, Wh, N, nullptr, act, nullptr, nullptr, N, nullptr, rowscale, s, &segs);
    }
}

// Gated pair (fp16 operands): the interleaved image has 64 rows per 32 outputs.
int64_t gated_image_rows(int64_t N) { return (N + 31) / 32 * 64; }
int launch_gemm16_gated(const uint16_t *x, int64_t M, int64_t K, const uint16_t *Wh, int64_t N, const float *bias, const float *bias2, int act,
                        float *y, const float *residual, const float *rowscale, hipStream_t s) {
    const int64_t rows = gated_image_rows(N);
    const bool big = pick_tile(M, rows) == 0;  // (the gated kernel exists for the two 128-column tiles)
    if (big && tile_env() != 1) return launch_gemm16_tile<false, 2, 2, true>(x, M, K, Wh, rows, bias, act, y, bias2, N, residual, rowscale, s);
    return launch_gemm16_tile<false, 1, 2, true>(x, M, K, Wh, rows, bias, act, y, bias2, N, residual, rowscale, s);
}

// Measured against the fused kernel (K = 4096, N = 4096 .. 14336): the two passes win from the
// first batch size the GEMV passes do not take (17 rows: 33 against 60 us for Q8_0 at 64 rows, 37
// against 66 .. 102 us at 512 rows) up to the largest.  The fused kernel comes within 5 % only for Q8_0 with bf16
// activations, whose conversion is the cheapest (2048 rows on 4096 x 4096: 79 us against 76 for the two passes; 1536 rows on
// 14336 -> 4096: 226 against 194); it serves the shapes the two passes do not take.
constexpr int64_t kMinRowsTwoPass = 17;
constexpr uint64_t kMaxImageBytes = (uint64_t)4 << 30;   // largest 16-bit weight image kept in a workspace

// GOMLX_HIPQ_TWO_PASS_MIN_ROWS=<rows> overrides the threshold (tuning runs only).
int64_t two_pass_env_rows() {
    static const int64_t v = [] { const char *e = std::getenv("GOMLX_HIPQ_TWO_PASS_MIN_ROWS"); return e ? (int64_t)std::atoll(e) : (int64_t)0; }();
    return v;
}

}  // namespace

// Per-thread byte offsets of a 256-row tile within 32 bits, 16-byte aligned activations.  The GEMM
// steps through K in 64s (whole LDS rows): bf16 activations are read in place and need K % 64 == 0,
// fp32 activations are rewritten anyway and get rows padded to that.
bool gemm_two_pass_supported(int type, bool x_is_bf16, int64_t M, int64_t K, int64_t N, const void *x) {
    if (type != kQ4_0 && type != kQ8_0 && type != kIQ4_NL && type != kQ4_K && type != kQ6_K) return false;
    const int64_t min_rows = two_pass_env_rows() > 0 ? two_pass_env_rows() : kMinRowsTwoPass;
    if (M < min_rows || K % (x_is_bf16 ? 64 : 32) != 0) return false;
    if (K > (1 << 22) || N > INT32_MAX || M > INT32_MAX || (M + 127) / 128 > 65535) return false;
    if ((uint64_t)N * (uint64_t)padded_k(K) * 2 > kMaxImageBytes) return false;
    return (reinterpret_cast<uintptr_t>(x) & 15) == 0;
}

// [16-bit weight image][fp32 activations only: fp16 activation image, M row scales][sums of the K slices, where K is split]
namespace {
size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
size_t two_pass_front_bytes(bool x_is_bf16, int64_t M, int64_t Kp, int64_t rows) {
    return align256((size_t)rows * Kp * 2) + (x_is_bf16 ? 0 : align256((size_t)M * Kp * 2) + align256((size_t)M * sizeof(float)));
}
}  // namespace
size_t gemm_two_pass_workspace(bool x_is_bf16, int64_t M, int64_t K, int64_t N) {
    K = padded_k(K);
    return two_pass_front_bytes(x_is_bf16, M, K, N) + gemm_partial_bytes(M, K, N);
}

int launch_gemm_two_pass(int type, bool x_is_bf16, const void *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias,
                         int act, float *y, void *workspace, hipStream_t s) {
    uint16_t *wh = static_cast<uint16_t *>(workspace);
    const int64_t Kp = padded_k(K);
    float *partial = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + two_pass_front_bytes(x_is_bf16, M, Kp, N));
    if (x_is_bf16) {
        if (int rc = launch_dequant16bit_type<true>(type, W, N, K, wh, s)) return rc;
        return launch_gemm16<true>(static_cast<const uint16_t *>(x), M, K, wh, N, bias, act, y, s, nullptr, nullptr, partial);
    }
    uint16_t *xh = wh + align256((size_t)N * Kp * 2) / 2;
    float *rowscale = reinterpret_cast<float *>(xh + align256((size_t)M * Kp * 2) / 2);
    if (int rc = launch_prep_f32(type, static_cast<const float *>(x), M, K, nullptr, xh, rowscale, prep_one_or_pair(W, nullptr, N), wh, s)) return rc;
    return launch_gemm16<false>(xh, M, Kp, wh, N, bias, act, y, s, nullptr, rowscale, partial);
}

// The two passes for a projection with its neighbours (fp32 activations): the RMS normalisation
// is folded into the activation pass, the residual into the GEMM's epilogue; a gated pair
// act(xn.W + bias) * (xn.W2 + bias2) is ONE GEMM over the interleaved image of both matrices, the
// product formed in registers, so neither projection is ever written out.
size_t gemm_two_pass_block_workspace(int64_t M, int64_t K, int64_t N, bool gated) {
    const int64_t rows = gated ? gated_image_rows(N) : N;
    K = padded_k(K);
    return two_pass_front_bytes(false, M, K, rows) + (gated ? 0 : gemm_partial_bytes(M, K, N));
}

bool gemm_two_pass_block_supported(int type, int64_t M, int64_t K, int64_t N, const void *x, bool gated) {
    if (!gemm_two_pass_supported(type, false, M, K, N, x)) return false;
    return !gated || (uint64_t)gated_image_rows(N) * (uint64_t)padded_k(K) * 2 <= kMaxImageBytes;
}

int launch_gemm_two_pass_block(int type, const float *x, int64_t M, int64_t K, const RmsNorm *norm, const uint8_t *W, const float *bias,
                               const uint8_t *W2, const float *bias2, const float *residual, int64_t N, int act, float *y, void *workspace,
                               hipStream_t s) {
    const int64_t rows = W2 ? gated_image_rows(N) : N;
    uint16_t *wh = static_cast<uint16_t *>(workspace);
    const int64_t Kp = padded_k(K);
    uint16_t *xh = wh + align256((size_t)rows * Kp * 2) / 2;
    float *rowscale = reinterpret_cast<float *>(xh + align256((size_t)M * Kp * 2) / 2);
    float *partial = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + two_pass_front_bytes(false, M, Kp, rows));
    if (int rc = launch_prep_f32(type, x, M, K, norm, xh, rowscale, prep_one_or_pair(W, W2, N), wh, s)) return rc;
    if (!W2) return launch_gemm16<false>(xh, M, Kp, wh, N, bias, act, y, s, residual, rowscale, partial);
    return launch_gemm16_gated(xh, M, Kp, wh, N, bias, bias2, act, y, residual, rowscale, s);
}

// Two to four matrices of one K against the same fp32 activations (the q / k / v projections behind one normalisation) at
// the batch sizes of the two-pass GEMM: the activations are converted ONCE, the matrices' images follow each other in
// one image, and ONE GEMM writes each matrix's columns to its own output - two launches where separate calls take six and
// convert the activations three times.  Every N a multiple of 32, one activation for all.
bool gemm_two_pass_set_supported(int type, int count, const MmqSetItem *items, int64_t M, int64_t K, const void *x) {
    if (count < 2 || count > 4) return false;
    int64_t ntot = 0;
    for (int i = 0; i < count; i++) {
        if (items[i].N <= 0 || items[i].N % 32 != 0 || items[i].act != items[0].act) return false;
        ntot += items[i].N;
    }
    return gemm_two_pass_supported(type, false, M, K, ntot, x);
}

size_t gemm_two_pass_set_workspace(int count, const MmqSetItem *items, int64_t M, int64_t K) {
    int64_t ntot = 0;
    for (int i = 0; i < count; i++) ntot += items[i].N;
    return gemm_two_pass_block_workspace(M, K, ntot, false);
}

int launch_gemm_two_pass_set(int type, const float *x, int64_t M, int64_t K, const RmsNorm *norm, int count, const MmqSetItem *items, void *workspace,
                             hipStream_t s) {
    PrepMatrices pm{};
    GemmSegs segs{};
    pm.count = segs.count = count;
    int64_t ntot = 0;
    for (int i = 0; i < count; i++) {
        pm.W[i] = items[i].W; pm.rows[i] = (uint32_t)items[i].N; pm.row0[i] = (uint32_t)ntot; pm.half[i] = 0;
        segs.y[i] = items[i].y; segs.bias[i] = items[i].bias; segs.n0[i] = (int)ntot;
        ntot += items[i].N;
    }
    segs.n0[count] = (int)ntot;
    uint16_t *wh = static_cast<uint16_t *>(workspace);
    const int64_t Kp = padded_k(K);
    uint16_t *xh = wh + align256((size_t)ntot * Kp * 2) / 2;
    float *rowscale = reinterpret_cast<float *>(xh + align256((size_t)M * Kp * 2) / 2);
    float *partial = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + two_pass_front_bytes(false, M, Kp, ntot));
    if (int rc = launch_prep_f32(type, x, M, K, norm, xh, rowscale, pm, wh, s)) return rc;
    return launch_gemm16_set(xh, M, Kp, wh, segs, items[0].act, rowscale, s, partial);
}

}  // namespace gq
