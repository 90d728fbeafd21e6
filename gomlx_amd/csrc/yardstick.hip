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

// Every workgroup reads ALL of a (small, cache-resident) buffer: the rate at which the L2 caches hand the same lines to all
// CUs at once, which is what a kernel pays that streams a shared operand past every workgroup.  DEPTH loads in flight per thread.
template <int DEPTH>
__global__ __launch_bounds__(1024) void read_shared_kernel(const uint4 *__restrict__ p, size_t chunks, int passes, uint32_t *__restrict__ out) {
    uint32_t acc = 0;
    for (int pass = 0; pass < passes; pass++) {
        size_t i = threadIdx.x;
        for (; i + (DEPTH - 1) * blockDim.x < chunks; i += DEPTH * blockDim.x) {
            uint4 v[DEPTH];
#pragma unroll
            for (int j = 0; j < DEPTH; j++) v[j] = p[i + j * blockDim.x];
#pragma unroll
            for (int j = 0; j < DEPTH; j++) acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
        }
        asm volatile("" : "+v"(acc));
    }
    if (acc == 0x9E3779B9u) out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc;
}

// The same shared buffer read the way a kernel with one stream per wavefront reads it: wavefront w of each workgroup takes
// the records w, w + 8, ... (`rec_bytes` each, a multiple of 4 KiB) and walks through them in 4 KiB pieces, three pieces in flight.
// DMA = false: ordinary 16-byte loads into registers; DMA = true: the same bytes by LDS DMA into a ring of four 4 KiB slots
// per wavefront (the way the small-batch kernels stage their activation image).  What differs between the two is the price
// of the LDS path alone.
template <bool DMA>
__global__ __launch_bounds__(512) void read_streams_kernel(const uint8_t *__restrict__ p, int records, int rec_bytes, uint32_t *__restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) uint8_t ring_lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pieces_per_rec = rec_bytes / 4096;
    const int my_recs = (records - wave + 7) / 8;
    const int total = my_recs * pieces_per_rec;  // pieces of this wavefront
    uint32_t acc = 0;
    auto piece_ptr = [&](int i) { return p + (size_t)(wave + 8 * (i / pieces_per_rec)) * rec_bytes + (size_t)(i % pieces_per_rec) * 4096 + lane * 16; };
    if constexpr (DMA) {
        uint8_t *ring = ring_lds + wave * 16384;
        auto issue = [&](int i) {
            const uint8_t *src = piece_ptr(i);
#pragma unroll
            for (int k = 0; k < 4; k++)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + k * 1024),
                                                 (__attribute__((address_space(3))) void *)(ring + (i & 3) * 4096 + k * 1024), 16, 0, 0);
        };
        for (int i = 0; i < 3 && i < total; i++) issue(i);
        for (int i = 0; i < total; i++) {
            if (i + 3 < total) {
                issue(i + 3);
                asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            const uint4 v = *reinterpret_cast<const uint4 *>(ring + (i & 3) * 4096 + lane * 16);
            acc ^= v.x ^ v.y ^ v.z ^ v.w;
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
    } else {
        uint4 v[4][4];
        auto issue = [&](int i, int slot) {
            const uint8_t *src = piece_ptr(i);
#pragma unroll
            for (int k = 0; k < 4; k++) v[slot][k] = *reinterpret_cast<const uint4 *>(src + k * 1024);
        };
        // (whole groups of four pieces keep the slots compile-time: records are 4 or 16 KiB multiples in the uses here)
        for (int i0 = 0; i0 < total; i0 += 4) {
#pragma unroll
            for (int j = 0; j < 4; j++) issue(min(i0 + j, total - 1), j);
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int k = 0; k < 4; k++) acc ^= v[j][k].x ^ v[j][k].y ^ v[j][k].z ^ v[j][k].w;
        }
    }
    if (acc == 0x9E3779B9u) out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc;
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

// gqy_mfma_valu: does vector-ALU work fit into the shadow of matrix instructions?  Every wavefront runs `groups` groups of
// four independent v_mfma_f32_32x32x16_bf16 (4 x 8 passes = 128 cycles of matrix work) plus NV independent vector-ALU
// instructions per group, either all behind the four matrix instructions (PLACE 0) or NV / 4 behind each of them
// (PLACE 1).  KIND picks the instruction: 0 v_fma_f32 (three register sources), 1 v_xor_b32 (two), 2 v_cvt_pk_bf16_f32.
// ACC: the accumulators live in 0 ordinary, 1 accumulation registers (AGPRs).
// The instruction order is pinned by volatile asm statements.  Every wavefront stamps the shader clock counter and the
// constant 100 MHz counter around its loop (clocks[(8 wg + wave) * 4 ..]): the span from a workgroup's first start to its
// last end, in shader cycles per group, is the figure of interest.  Workgroups of 256 threads put one wavefront on each SIMD
// (128 cycles of matrix work per group), of 512 two (256 cycles; the two do not share a SIMD evenly - the older one
// finishes first - which is why the span over all wavefronts is taken).  Free vector-ALU work leaves the figure at the
// matrix cycles; 4 more cycles per instruction mean that nothing overlaps.
template <int NV, int PLACE, int KIND, int ACC>
__global__ __launch_bounds__(512) void mfma_valu_kernel(const uint4 *__restrict__ frags, int groups, unsigned long long *__restrict__ clocks,
                                                        float *__restrict__ sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    bf16x8 a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        a[i] = __builtin_bit_cast(bf16x8, frags[(wave * 4 + i) * 64 + lane]);
        b[i] = __builtin_bit_cast(bf16x8, frags[(wave * 4 + 2 + i) * 64 + lane]);
    }
    f32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
    constexpr int NT = 12;  // independent vector-ALU chains (an instruction depends on the one NT before it)
    float t[NT];
#pragma unroll
    for (int i = 0; i < NT; i++) t[i] = 1.0f + (float)(lane + i) * 1e-3f;
    float c1 = 1.0000001f, c2 = 1e-9f;
    asm volatile("" : "+v"(c1), "+v"(c2));
    unsigned long long *stamp = clocks + ((size_t)blockIdx.x * 8 + wave) * 4;
    if (lane == 0) {
        stamp[0] = clock64();
        stamp[1] = wall_clock64();
    }
    auto valu = [&](int n) __attribute__((always_inline)) {
        float &x = t[n % NT];
        if constexpr (KIND == 0) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x) : "v"(c1), "v"(c2));
        else if constexpr (KIND == 1) asm volatile("v_xor_b32 %0, %0, %1" : "+v"(x) : "v"(c2));
        else asm volatile("v_cvt_pk_bf16_f32 %0, %0, %1" : "+v"(x) : "v"(c1));
    };
    for (int g = 0; g < groups; g++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if constexpr (ACC == 1) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a[i & 1]), "v"(b[i >> 1]));
            else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a[i & 1]), "v"(b[i >> 1]));
            if constexpr (PLACE == 1) {
#pragma unroll
                for (int n = 0; n < NV / 4; n++) valu(i * (NV / 4) + n);
            }
        }
        if constexpr (PLACE == 0) {
#pragma unroll
            for (int n = 0; n < NV; n++) valu(n);
        }
    }
    float r = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int k = 0; k < 16; k++) r += acc[i][k];
#pragma unroll
    for (int i = 0; i < NT; i++) r += t[i];
    if (lane == 0) {
        stamp[2] = clock64() + (r == 12345.678f ? 1 : 0);
        stamp[3] = wall_clock64();
    }
    if (r == 12345.678f) sink[blockIdx.x * 512 + threadIdx.x] = r;
}

template <int NV, int PLACE, int ACC>
int launch_mfma_valu(int kind, const uint4 *frags, int groups, int wgs, int threads, unsigned long long *clocks, float *sink, hipStream_t s) {
    switch (kind) {
    case 0: hipLaunchKernelGGL((mfma_valu_kernel<NV, PLACE, 0, ACC>), dim3(wgs), dim3(threads), 0, s, frags, groups, clocks, sink); break;
    case 1: hipLaunchKernelGGL((mfma_valu_kernel<NV, PLACE, 1, ACC>), dim3(wgs), dim3(threads), 0, s, frags, groups, clocks, sink); break;
    default: hipLaunchKernelGGL((mfma_valu_kernel<NV, PLACE, 2, ACC>), dim3(wgs), dim3(threads), 0, s, frags, groups, clocks, sink); break;
    }
    return (int)hipGetLastError();
}

}  // namespace

extern "C" {

// nv in {0, 8, 16, 32, 48}; place 0 (behind the group) or 1 (interleaved); kind 0 / 1 / 2 (fma / xor / pack to bf16);
// acc 0 (accumulators in ordinary registers) or 1 (in accumulation registers); threads 256 (one wavefront per SIMD) or
// 512 (two).  frags and sink as for gqy_mfma; clocks: 32 x wgs uint64 (four stamps per wavefront).  Returns 0, -1 for bad
// arguments, or a hipError_t.
int gqy_mfma_valu(const void *frags, int groups, int wgs, int threads, int nv, int place, int kind, int acc, void *clocks, void *sink, void *stream) {
    const uint4 *f = static_cast<const uint4 *>(frags);
    unsigned long long *c = static_cast<unsigned long long *>(clocks);
    float *k = static_cast<float *>(sink);
    hipStream_t s = (hipStream_t)stream;
    if ((threads != 256 && threads != 512) || (place != 0 && place != 1) || kind < 0 || kind > 2 || (acc != 0 && acc != 1)) return -1;
#define GQY_CASE(NV)                                                                                                              \
    case NV:                                                                                                                      \
        if (acc) return place ? launch_mfma_valu<NV, 1, 1>(kind, f, groups, wgs, threads, c, k, s) : launch_mfma_valu<NV, 0, 1>(kind, f, groups, wgs, threads, c, k, s); \
        return place ? launch_mfma_valu<NV, 1, 0>(kind, f, groups, wgs, threads, c, k, s) : launch_mfma_valu<NV, 0, 0>(kind, f, groups, wgs, threads, c, k, s);
    switch (nv) {
        GQY_CASE(0)
        GQY_CASE(8)
        GQY_CASE(16)
        GQY_CASE(32)
        GQY_CASE(48)
    default: return -1;
    }
#undef GQY_CASE
}

// frags: 8 wavefronts x 4 fragments x 64 lanes x 16 bytes (32 KiB) of bf16 operands; clocks: 4 x wgs uint64; sink: wgs x 512 floats.
// Each wavefront issues 4 * groups matrix instructions (2 * 32 * 32 * 16 flop each).  Returns 0 or a hipError_t.
int gqy_mfma(const void *frags, int groups, int wgs, void *clocks, void *sink, void *stream) {
    hipLaunchKernelGGL(mfma_only_kernel, dim3(wgs), dim3(512), 0, (hipStream_t)stream, static_cast<const uint4 *>(frags), groups,
                       static_cast<unsigned long long *>(clocks), static_cast<float *>(sink));
    return (int)hipGetLastError();
}

// Every one of `wgs` workgroups of `threads` threads reads the whole buffer `passes` times, 8 loads in flight per thread.
int gqy_read_shared(const void *p, size_t bytes, int wgs, int threads, int passes, void *out, void *stream) {
    hipLaunchKernelGGL(read_shared_kernel<8>, dim3(wgs), dim3(threads), 0, (hipStream_t)stream, static_cast<const uint4 *>(p), bytes / 16, passes,
                       static_cast<uint32_t *>(out));
    return (int)hipGetLastError();
}

// Every one of `wgs` workgroups (512 threads) reads `records` records of rec_bytes, one stream per wavefront; dma 0 / 1.
int gqy_read_streams(const void *p, int records, int rec_bytes, int wgs, int dma, void *out, void *stream) {
    if (rec_bytes % 4096 != 0 || records < 8) return -1;
    if (dma) {
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(read_streams_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, 8 * 16384);
        if (attr != hipSuccess) return (int)attr;
        hipLaunchKernelGGL(read_streams_kernel<true>, dim3(wgs), dim3(512), 8 * 16384, (hipStream_t)stream, static_cast<const uint8_t *>(p), records, rec_bytes,
                           static_cast<uint32_t *>(out));
    } else {
        hipLaunchKernelGGL(read_streams_kernel<false>, dim3(wgs), dim3(512), 0, (hipStream_t)stream, static_cast<const uint8_t *>(p), records, rec_bytes,
                           static_cast<uint32_t *>(out));
    }
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
