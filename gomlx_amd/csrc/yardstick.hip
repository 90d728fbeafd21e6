// Read-only streaming kernels of known size: the yardsticks the decode kernels are judged against.
// Built into libgq_yardstick.so, which only the benchmark loads (nothing in libgomlx_hipq.so uses it).
//
//   gqy_read(pattern 0): every byte of a buffer is loaded once with 16-byte loads, consecutive lanes on
//     consecutive chunks, by `wgs` workgroups of `threads` threads; each thread keeps `depth` loads in
//     flight and folds what arrives into one xor (so nothing is optimised away); no other arithmetic,
//     one 4-byte store per thread at the end.  This is the time in which this chip hands a one-shot
//     kernel that many cold bytes: what a bandwidth-bound kernel of the same grid can reach at best.
//   gqy_read(pattern 1, 2): the same bytes of a Q4_K matrix [N, row_bytes] read the way the small-batch
//     kernel's wavefronts address them: 32 rows x one 144-byte super-block per wavefront step,
//     (1) one row per lane pair (header + four 16-byte pieces per lane: each load instruction touches
//     32 different rows), (2) as consecutive 16-byte chunks of a row (nine per row, seven rows per
//     load instruction).  The difference between 1 and 2 is the price of the address pattern alone.
//   gqy_mfma: matrix instructions and nothing else.  Every wavefront of `wgs` workgroups (8 wavefronts each, two per
//     SIMD, the prefill GEMM's occupancy) loads four operand fragments once and then issues `groups` groups of four
//     independent v_mfma_f32_32x32x16_bf16 on its four accumulators: no memory traffic, no LDS, no barrier, no
//     vector-ALU work inside the loop.  Each workgroup also reads the shader clock counter and the constant
//     100 MHz counter before and after its loop, which gives the clock the chip actually ran at.  This is the rate at
//     which this chip issues that many matrix instructions under its power limit: the ceiling for a GEMM of the
//     same instruction count, whatever its data movement costs.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <int DEPTH, bool NT = false>
__global__ __launch_bounds__(1024) void read_linear_kernel(const uint4 *__restrict__ p, size_t chunks, uint32_t *__restrict__ out) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t acc = 0;
    for (; i + (DEPTH - 1) * stride < chunks; i += DEPTH * stride) {
        uint4 v[DEPTH];
#pragma unroll
        for (int j = 0; j < DEPTH; j++) {
            if constexpr (NT) {  // non-temporal: the line is not kept in the caches behind the load
                const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p + i + j * stride));
                v[j] = make_uint4(t.x, t.y, t.z, t.w);
            } else v[j] = p[i + j * stride];
        }
#pragma unroll
        for (int j = 0; j < DEPTH; j++) acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
    }
    for (; i < chunks; i += stride) { const uint4 v = p[i]; acc ^= v.x ^ v.y ^ v.z ^ v.w; }
    if (acc == 0x9E3779B9u) out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc;  // (practically never: keeps the loads alive)
}

// grid (N / 128, slices); 512 threads: wavefront = (row tile of 32, half of the slice's super-blocks), all loads up front
template <bool COALESCED>
__global__ __launch_bounds__(512) void read_q4k_tiles_kernel(const uint8_t *__restrict__ W, int N, int64_t row_bytes, int slice_sb, int sbs,
                                                             uint32_t *__restrict__ out) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rt = wave & 3, par = wave >> 2;
    const int sb0 = blockIdx.y * slice_sb;
    const int nsb = min(slice_sb, sbs - sb0);
    const int row0 = blockIdx.x * 128 + rt * 32;
    uint32_t acc = 0;
    uint4 v[4][5];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int sb = sb0 + min(par + 2 * i, nsb - 1);
        if constexpr (COALESCED) {
#pragma unroll
            for (int l = 0; l < 5; l++) {
                const int c = min(lane + 64 * l, 32 * 9 - 1);
                v[i][l] = *reinterpret_cast<const uint4 *>(W + (int64_t)min(row0 + c / 9, N - 1) * row_bytes + (int64_t)sb * 144 + (c % 9) * 16);
            }
        } else {
            const uint8_t *p = W + (int64_t)min(row0 + (lane & 31), N - 1) * row_bytes + (int64_t)sb * 144;
            v[i][0] = *reinterpret_cast<const uint4 *>(p);
#pragma unroll
            for (int l = 0; l < 4; l++) v[i][1 + l] = *reinterpret_cast<const uint4 *>(p + 16 + 32 * l + 16 * (lane >> 5));
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int l = 0; l < 5; l++) acc ^= v[i][l].x ^ v[i][l].y ^ v[i][l].z ^ v[i][l].w;
    if (acc == 0x9E3779B9u) out[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 512 + tid] = acc;
}

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// clocks[4 wg .. 4 wg + 3] = shader clock at start, 100 MHz clock at start, shader clock at end, 100 MHz clock at end
__global__ __launch_bounds__(512) void mfma_only_kernel(const uint4 *__restrict__ frags, int groups, unsigned long long *__restrict__ clocks,
                                                        float *__restrict__ sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    bf16x8 a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        a[i] = __builtin_bit_cast(bf16x8, frags[(wave * 4 + i) * 64 + lane]);
        b[i] = __builtin_bit_cast(bf16x8, frags[(wave * 4 + 2 + i) * 64 + lane]);
    }
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    if (threadIdx.x == 0) {
        clocks[4 * blockIdx.x] = clock64();
        clocks[4 * blockIdx.x + 1] = wall_clock64();
    }
    for (int g = 0; g < groups; g++) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) t += acc[i][j][r];
    // (wavefront 0's last accumulator is read above: the end stamp is taken after its matrix instructions have completed)
    if (threadIdx.x == 0) {
        clocks[4 * blockIdx.x + 2] = clock64() + (t == 12345.678f ? 1 : 0);
        clocks[4 * blockIdx.x + 3] = wall_clock64();
    }
    if (t == 12345.678f) sink[blockIdx.x * 512 + threadIdx.x] = t;  // (practically never: keeps the instructions alive)
}

}  // namespace

extern "C" {

// frags: 8 wavefronts x 4 fragments x 64 lanes x 16 bytes (32 KiB) of bf16 operands; clocks: 4 x wgs uint64; sink: wgs x 512 floats.
// Each wavefront issues 4 * groups matrix instructions (2 * 32 * 32 * 16 flop each).  Returns 0 or a hipError_t.
int gqy_mfma(const void *frags, int groups, int wgs, void *clocks, void *sink, void *stream) {
    hipLaunchKernelGGL(mfma_only_kernel, dim3(wgs), dim3(512), 0, (hipStream_t)stream, static_cast<const uint4 *>(frags), groups,
                       static_cast<unsigned long long *>(clocks), static_cast<float *>(sink));
    return (int)hipGetLastError();
}

// pattern 0: linear (N, row_bytes, slice_sb ignored).  pattern 1 / 2: Q4_K tiles, row per lane / coalesced.
// `out` must hold wgs * threads (pattern 0) or (N / 128) * slices * 512 (patterns 1, 2) uint32.  Returns 0 or a hipError_t.
int gqy_read(const void *p, size_t bytes, int pattern, int wgs, int threads, int depth, int64_t N, int64_t row_bytes, int slice_sb,
             void *out, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (pattern == 0) {
        const size_t chunks = bytes / 16;
        const uint4 *q = static_cast<const uint4 *>(p);
        uint32_t *o = static_cast<uint32_t *>(out);
        if (pattern == 0 && depth >= 100) {  // depth 102 / 104 / 108: non-temporal loads, 2 / 4 / 8 in flight
            switch (depth - 100) {
            case 2: hipLaunchKernelGGL((read_linear_kernel<2, true>), dim3(wgs), dim3(threads), 0, s, q, chunks, o); break;
            case 4: hipLaunchKernelGGL((read_linear_kernel<4, true>), dim3(wgs), dim3(threads), 0, s, q, chunks, o); break;
            default: hipLaunchKernelGGL((read_linear_kernel<8, true>), dim3(wgs), dim3(threads), 0, s, q, chunks, o); break;
            }
            return (int)hipGetLastError();
        }
        switch (depth) {
        case 1: hipLaunchKernelGGL(read_linear_kernel<1>, dim3(wgs), dim3(threads), 0, s, q, chunks, o); break;
        case 2: hipLaunchKernelGGL(read_linear_kernel<2>, dim3(wgs), dim3(threads), 0, s, q, chunks, o); break;
        case 4: hipLaunchKernelGGL(read_linear_kernel<4>, dim3(wgs), dim3(threads), 0, s, q, chunks, o); break;
        case 8: hipLaunchKernelGGL(read_linear_kernel<8>, dim3(wgs), dim3(threads), 0, s, q, chunks, o); break;
        default: hipLaunchKernelGGL(read_linear_kernel<16>, dim3(wgs), dim3(threads), 0, s, q, chunks, o); break;
        }
    } else {
        const int sbs = (int)(row_bytes / 144);
        const dim3 grid((unsigned)((N + 127) / 128), (unsigned)((sbs + slice_sb - 1) / slice_sb));
        if (pattern == 2)
            hipLaunchKernelGGL(read_q4k_tiles_kernel<true>, grid, dim3(512), 0, s, static_cast<const uint8_t *>(p), (int)N, row_bytes, slice_sb, sbs,
                               static_cast<uint32_t *>(out));
        else
            hipLaunchKernelGGL(read_q4k_tiles_kernel<false>, grid, dim3(512), 0, s, static_cast<const uint8_t *>(p), (int)N, row_bytes, slice_sb, sbs,
                               static_cast<uint32_t *>(out));
    }
    return (int)hipGetLastError();
}

}  // extern "C"
