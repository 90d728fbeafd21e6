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
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

template <int DEPTH>
__global__ __launch_bounds__(1024) void read_linear_kernel(const uint4 *__restrict__ p, size_t chunks, uint32_t *__restrict__ out) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t acc = 0;
    for (; i + (DEPTH - 1) * stride < chunks; i += DEPTH * stride) {
        uint4 v[DEPTH];
#pragma unroll
        for (int j = 0; j < DEPTH; j++) v[j] = p[i + j * stride];
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

}  // namespace

extern "C" {

// pattern 0: linear (N, row_bytes, slice_sb ignored).  pattern 1 / 2: Q4_K tiles, row per lane / coalesced.
// `out` must hold wgs * threads (pattern 0) or (N / 128) * slices * 512 (patterns 1, 2) uint32.  Returns 0 or a hipError_t.
int gqy_read(const void *p, size_t bytes, int pattern, int wgs, int threads, int depth, int64_t N, int64_t row_bytes, int slice_sb,
             void *out, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    if (pattern == 0) {
        const size_t chunks = bytes / 16;
        const uint4 *q = static_cast<const uint4 *>(p);
        uint32_t *o = static_cast<uint32_t *>(out);
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
