// Small-batch (decode batch 5..~128) quantised Dense for Q4_K on the gfx950 matrix cores.
//
// At batch 32 the contraction is 228 flop per weight byte: far beyond the vector ALUs, still
// below the MFMA machine balance, so the kernel should run at the speed the packed weights
// stream from HBM.  Two things decide whether it does:
//
//  * Activation traffic.  Every 16-row tile of W needs all of x.  Fetching x per tile through
//    the CU's vector-memory path would move ~7x more bytes than the weights themselves, so the
//    work is split along K instead: a workgroup owns a K-slice of 2048 values (8 super-blocks),
//    keeps the slice of x for 32 batch columns resident in LDS (fp16, 128 KiB) and streams
//    128 rows of W past it.  Slices are summed by a second, tiny kernel that also applies
//    bias and activation (deterministic order, no atomics).
//
//  * VALU work per weight.  Codes are never dequantised to fp32.  A 16-byte run of code bytes
//    becomes four MFMA operand fragments directly in registers: (dword & 0x000F000F) | 0x6400
//    is the fp16 pair (1024 + n_a, 1024 + n_b); one packed fma with the 6-bit sub-block scale
//    gives the exact integers sc*n (<= 945, exact in fp16); these accumulate over a whole
//    super-block on v_mfma_f32_16x16x32_f16, and only then are scaled by the fp16 d in fp32.
//    The sub-block minima ride on one extra MFMA per super-block against per-sub-block sums
//    of x.  The only rounding that is not fp32 is x -> fp16 (2^-12 relative).
//
// MFMA roles: A = activations (rows = batch columns), B = weights (columns = W rows), so a
// lane's four results belong to ONE weight row, the one whose header it has already loaded.
#include "blocks.hpp"
#include "common.hpp"

#include <map>
#include <mutex>

namespace gq {

namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int kSliceSB = 8;                 // super-blocks per K-slice
constexpr int kSliceK = kSliceSB * 256;     // 2048 values
constexpr int kRowsPerWG = 128;             // 8 wavefronts x 16 rows
constexpr int kMT = 32;                     // batch columns per pass
constexpr int kXFBytes = kSliceK * kMT * 2;          // 131072: fp16 activations, fragment order
constexpr int kXSBytes = kSliceSB * 2 * kMT * 8;     // 4096: sub-block sums, fragment order
constexpr int kLdsBytes = kXFBytes + kXSBytes;

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    h2 v;
    v.x = (_Float16)a;
    v.y = (_Float16)b;
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }

// (u & mask) | 0x64006400 as an fp16 pair: 1024 + n (mask 0x000F000F) or 1024 + 16 n (0x00F000F0)
__device__ __forceinline__ h2 magic_pair(uint32_t u, uint32_t mask) { return as_h2((u & mask) | 0x64006400u); }

__device__ __forceinline__ float dpp_quad_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    return v;
}

// ---- stage the K-slice of x into LDS in MFMA fragment order ---------------------------------
//
// One item = 8 consecutive activations of one batch column ("octet").  Inside a super-block the
// value index v = 64 g' + 32 high + idx: byte idx of group g', low (high = 0) or high nibble.
// A lane of the main loop loads the 16-byte chunk c = 2 g' + idx / 16 and turns it into four
// octets q = 2 high + (idx % 16) / 8; chunk c is handled at step t = c / 4 by lane group
// g = c % 4.  Within an octet the code bytes come out in the order (0, 2, 1, 3, 4, 6, 5, 7).
__device__ __forceinline__ void stage_x(const float *__restrict__ X, int M, int K, int m0, int k0, uint8_t *lds, int tid) {
    constexpr int kItems = kMT * (kSliceK / 8);  // 8192
    constexpr int kBatch = 4;
    for (int base = 0; base < kItems; base += 512 * kBatch) {
        float4 lo[kBatch], hi[kBatch];
#pragma unroll
        for (int r = 0; r < kBatch; r++) {
            const int i = base + r * 512 + tid;
            const int m = i >> 8, oct = i & 255;
            const int k = k0 + 8 * oct;
            const bool ok = (m0 + m < M) && (k < K);
            const float4 *p = reinterpret_cast<const float4 *>(X + (int64_t)min(m0 + m, M - 1) * K + min(k, K - 8));
            const float4 a = p[0], b = p[1];
            lo[r] = ok ? a : make_float4(0.f, 0.f, 0.f, 0.f);
            hi[r] = ok ? b : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int r = 0; r < kBatch; r++) {
            const int i = base + r * 512 + tid;
            const int m = i >> 8, oct = i & 255;
            const int sbl = oct >> 5, v8 = oct & 31;
            const int gp = v8 >> 3, w8 = v8 & 7, high = w8 >> 2, idx8 = w8 & 3;
            const int q = high * 2 + (idx8 & 1);
            const int c = 2 * gp + (idx8 >> 1);
            const int t = c >> 2, g = c & 3;
            const float4 a = lo[r], b = hi[r];
            uint4 o;  // bytes (0,2,1,3,4,6,5,7)
            o.x = pack_h2(a.x, a.z);
            o.y = pack_h2(a.y, a.w);
            o.z = pack_h2(b.x, b.z);
            o.w = pack_h2(b.y, b.w);
            *reinterpret_cast<uint4 *>(lds + ((((sbl * 2 + t) * 4 + q) * 4 + g) * kMT + m) * 16) = o;
            float s = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w));
            s = dpp_quad_sum(s);  // the four octets of one 32-value sub-block sit in one quad
            if ((oct & 3) == 0) {
                const int j = 2 * gp + high;
                const int gsel = (j >> 1) & 1, pos = (j & 1) + 2 * (j >> 2);
                *reinterpret_cast<_Float16 *>(lds + kXFBytes + (((sbl * 2 + gsel) * kMT + m) * 4 + pos) * 2) = (_Float16)s;
            }
        }
    }
}

struct RawSB { uint4 hd, c0, c1; };  // header + this lane's chunk at step 0 and step 1

__device__ __forceinline__ void load_sb(RawSB &r, const uint8_t *sb, int g) {
    r.hd = *reinterpret_cast<const uint4 *>(sb);
    r.c0 = *reinterpret_cast<const uint4 *>(sb + 16 + 16 * g);
    r.c1 = *reinterpret_cast<const uint4 *>(sb + 16 + 64 + 16 * g);
}

// partial[slice][m][n] = sum over the slice's k of x[m][k] * w[n][k]
__global__ __launch_bounds__(512) void mmq_q4k_kernel(const float *__restrict__ X, const uint8_t *__restrict__ W,
                                                      float *__restrict__ partial, int M, int K, int N,
                                                      int64_t row_bytes, int m0) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, col = lane & 15;
    const int slice = blockIdx.y;
    const int k0 = slice * kSliceK;
    const int nsb = min(kSliceSB, (K - k0) >> 8);
    const int n = blockIdx.x * kRowsPerWG + wave * 16 + col;  // this lane's weight row
    const uint8_t *wrow = W + (int64_t)min(n, N - 1) * row_bytes + (int64_t)(k0 >> 8) * 144;

    RawSB cur, nxt;
    load_sb(cur, wrow, g);
    stage_x(X, M, K, m0, k0, lds, tid);
    __syncthreads();

    f4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    const uint8_t *xf = lds + (g * kMT + col) * 16;   // + ((sbl*2+t)*4+q) * (4*kMT*16) + half*256
    const uint8_t *xs = lds + kXFBytes + ((g >> 1) * kMT + col) * 8;  // + sbl * (2*kMT*8) + half*128

    for (int sbl = 0; sbl < nsb; sbl++) {
        load_sb(nxt, wrow + (int64_t)min(sbl + 1, nsb - 1) * 144, g);
        const float d = half_bits_to_float(cur.hd.x & 0xFFFFu), dmin = half_bits_to_float(cur.hd.x >> 16);
        // all eight 6-bit scales / minima as bytes: sc0..3, sc4..7, m0..3, m4..7
        const uint32_t a = cur.hd.y, b = cur.hd.z, c = cur.hd.w;
        const uint32_t sc_lo = a & 0x3F3F3F3Fu, mn_lo = b & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (c & 0x0F0F0F0Fu) | ((a >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((c >> 4) & 0x0F0F0F0Fu) | ((b >> 2) & 0x30303030u);
        f4 p1[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int t = 0; t < 2; t++) {
            // chunk 4t+g: group g' = 2t + g/2, sub-blocks j0 = 2g' (low nibbles), j0+1 (high nibbles)
            const uint32_t scw = (t == 0 ? sc_lo : sc_hi) >> (16 * (g >> 1));
            const float s0f = (float)(scw & 0xFFu), s1f = (float)((scw >> 8) & 0xFFu);
            const h2 s0 = as_h2(pack_h2(s0f, s0f));
            const h2 s1 = as_h2(pack_h2(s1f * 0.0625f, s1f * 0.0625f));  // high-nibble pairs arrive as 1024 + 16 n
            const h2 k0h = as_h2(pack_h2(-1024.f * s0f, -1024.f * s0f));
            const h2 k1h = as_h2(pack_h2(-64.f * s1f, -64.f * s1f));
            const uint4 ch = t == 0 ? cur.c0 : cur.c1;
            const uint32_t dw[4] = {ch.x, ch.y, ch.z, ch.w};
            uint32_t wl[8], wh[8];
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t u = dw[w], v = dw[w] >> 8;
                wl[2 * w] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(u, 0x000F000Fu), s0, k0h));
                wl[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(v, 0x000F000Fu), s0, k0h));
                wh[2 * w] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(u, 0x00F000F0u), s1, k1h));
                wh[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(magic_pair(v, 0x00F000F0u), s1, k1h));
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t *src = (q < 2 ? wl : wh) + 4 * (q & 1);
                const uint4 wv = make_uint4(src[0], src[1], src[2], src[3]);
                const h8 wfrag = __builtin_bit_cast(h8, wv);
                const uint8_t *xp = xf + ((sbl * 2 + t) * 4 + q) * (4 * kMT * 16);
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const h8 xfrag = *reinterpret_cast<const h8 *>(xp + h * 256);
                    p1[h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xfrag, wfrag, p1[h], 0, 0, 0);
                }
            }
        }
        // minima: lane groups 0 and 2 carry (m0,m1,m4,m5) and (m2,m3,m6,m7) against the matching sums
        uint4 mv = make_uint4(0u, 0u, 0u, 0u);
        if ((g & 1) == 0) {
            const int sh = 16 * (g >> 1);
            const uint32_t lo2 = mn_lo >> sh, hi2 = mn_hi >> sh;
            mv.x = pack_h2((float)(lo2 & 0xFFu), (float)((lo2 >> 8) & 0xFFu));
            mv.y = pack_h2((float)(hi2 & 0xFFu), (float)((hi2 >> 8) & 0xFFu));
        }
        const h8 mfrag = __builtin_bit_cast(h8, mv);
        f4 p2[2];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint4 sv = make_uint4(0u, 0u, 0u, 0u);
            if ((g & 1) == 0) {
                const uint2 s2 = *reinterpret_cast<const uint2 *>(xs + sbl * (2 * kMT * 8) + h * 128);
                sv.x = s2.x;
                sv.y = s2.y;
            }
            const f4 zero = {0.f, 0.f, 0.f, 0.f};
            p2[h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, sv), mfrag, zero, 0, 0, 0);
        }
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[h][r] = fmaf(d, p1[h][r], fmaf(-dmin, p2[h][r], acc[h][r]));
        cur = nxt;
    }

    // lane holds y[m = 16 h + 4 g + r][n] for its K-slice
    if (n < N) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int m = m0 + 16 * h + 4 * g + r;
                if (m < M) partial[((int64_t)slice * M + m) * N + n] = acc[h][r];
            }
    }
}

// y[m][n] = act(sum_s partial[s][m][n] + bias[n])
__global__ __launch_bounds__(256) void mmq_reduce_kernel(const float *__restrict__ partial, int nslices, int64_t MN, int N,
                                                         const float *__restrict__ bias, int act, float *__restrict__ Y) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < MN; i += (int64_t)gridDim.x * 256) {
        float s = 0.f;
        for (int k = 0; k < nslices; k++) s += partial[(int64_t)k * MN + i];
        if (bias) s += bias[i % N];
        Y[i] = apply_act(act, s);
    }
}

// ---- per-stream workspace for the K-slice partial sums -----------------------------------
struct Workspace { void *ptr = nullptr; size_t bytes = 0; };
std::mutex g_ws_mutex;
std::map<hipStream_t, Workspace> g_ws;

int workspace_for(hipStream_t s, size_t bytes, float **out) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace &w = g_ws[s];
    if (w.bytes < bytes) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (s != nullptr && hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone)
            return fail(GQ_ERR_INVALID, "qdense: the %zu-byte split-K workspace of this stream must exist before a graph is "
                        "recorded; run the same call once outside the recording first", bytes);
        // An outgrown buffer is retired, not freed: a recorded graph may still point at it.
        w = Workspace();
        size_t want = bytes < (size_t)(4u << 20) ? (size_t)(4u << 20) : bytes;
        GQ_HIP(hipMalloc(&w.ptr, want));
        w.bytes = want;
    }
    *out = static_cast<float *>(w.ptr);
    return GQ_OK;
}

}  // namespace

bool mmq_supported(int type, int64_t M, int64_t K, int64_t N, const void *x) {
    return type == kQ4_K && M >= 2 && M <= 256 && K % 256 == 0 && N <= (int64_t)INT32_MAX / 2 && K <= INT32_MAX &&
           (reinterpret_cast<uintptr_t>(x) & 15) == 0;
}

int launch_mmq(int type, const float *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act,
               float *y, hipStream_t s) {
    if (type != kQ4_K) return fail(GQ_ERR_NOT_IMPLEMENTED, "mmq: ggml type %d is not implemented", type);
    static const bool lds_ok = [] {
        return hipFuncSetAttribute(reinterpret_cast<const void *>(mmq_q4k_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   kLdsBytes) == hipSuccess;
    }();
    if (!lds_ok) return fail(GQ_ERR_HIP, "mmq: cannot reserve %d bytes of LDS", kLdsBytes);
    const int nslices = (int)((K + kSliceK - 1) / kSliceK);
    float *partial = nullptr;
    if (int rc = workspace_for(s, (size_t)nslices * M * N * sizeof(float), &partial)) return rc;
    const int64_t row_bytes = (K / 256) * 144;
    const dim3 grid((unsigned)((N + kRowsPerWG - 1) / kRowsPerWG), (unsigned)nslices);
    for (int64_t m0 = 0; m0 < M; m0 += kMT) {
        if (int rc = launch(mmq_q4k_kernel, grid, dim3(512), (size_t)kLdsBytes, s, x, W, partial, (int)M, (int)K, (int)N,
                            row_bytes, (int)m0))
            return rc;
    }
    const int64_t MN = M * N;
    int64_t blocks = (MN + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    return launch(mmq_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const float *)partial, nslices, MN, (int)N, bias,
                  act, y);
}

}  // namespace gq
