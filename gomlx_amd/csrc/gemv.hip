// Decode GEMV for GGML-quantised weights on gfx950: y[n] = act(sum_k x[k] * w[n,k] + b[n]).
//
// Bandwidth-bound: the only HBM traffic that matters is one pass over the packed weight
// rows.  Each lane owns one 32-value block (Q4_0 / Q8_0 / IQ4_NL) or one eighth of a
// 256-value super-block (Q4_K) per step, fetches its packed codes with 16-byte loads that
// are contiguous across the wavefront, decodes them in registers (v_cvt_f32_ubyteN on
// masked dwords), multiplies with activations held in LDS in a lane-major layout, and the
// R rows a wavefront works on are reduced with DPP / cross-row shuffles at the end.
// The block scale is applied once per block, and the constant code offset (-8 for Q4_0,
// +128 bias trick for the signed Q8_0 bytes, the Q4_K minimum) is folded into a per-block
// sum of x that is shared by all R rows.
#include "blocks.hpp"
#include "common.hpp"

namespace gq {

namespace {

// ---- per-format register images of one lane's share of a row -------------------------------

template <int T> struct LaneBlock;

template <> struct LaneBlock<kQ4_0> {
    uint32_t d;
    u128_a2 q;
    __device__ __forceinline__ void load(const uint8_t *p) {
        d = load_u16(p);
        q = *reinterpret_cast<const u128_a2 *>(p + 2);
    }
    // sum_i (nib_i - 8) * x_i * d
    __device__ __forceinline__ float dot(const float *xv, float xsum) const {
        float lo = 0.f, hi = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t l = q.v[w] & 0x0F0F0F0Fu, h = q.v[w] & 0xF0F0F0F0u;  // h holds 16 * nibble
            lo = fmaf(ubyte0(l), xv[4 * w + 0], lo);
            lo = fmaf(ubyte1(l), xv[4 * w + 1], lo);
            lo = fmaf(ubyte2(l), xv[4 * w + 2], lo);
            lo = fmaf(ubyte3(l), xv[4 * w + 3], lo);
            hi = fmaf(ubyte0(h), xv[16 + 4 * w + 0], hi);
            hi = fmaf(ubyte1(h), xv[16 + 4 * w + 1], hi);
            hi = fmaf(ubyte2(h), xv[16 + 4 * w + 2], hi);
            hi = fmaf(ubyte3(h), xv[16 + 4 * w + 3], hi);
        }
        return half_bits_to_float(d) * (fmaf(hi, 0.0625f, lo) - 8.0f * xsum);
    }
};

template <> struct LaneBlock<kIQ4_NL> {
    uint32_t d;
    u128_a2 q;
    __device__ __forceinline__ void load(const uint8_t *p) {
        d = load_u16(p);
        q = *reinterpret_cast<const u128_a2 *>(p + 2);
    }
    __device__ __forceinline__ float dot(const float *xv, float) const {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t b = (q.v[w] >> (8 * j)) & 0xFFu;
                s = fmaf(iq4nl_value(b & 15u), xv[4 * w + j], s);
                s = fmaf(iq4nl_value(b >> 4), xv[16 + 4 * w + j], s);
            }
        }
        return half_bits_to_float(d) * s;
    }
};

template <> struct LaneBlock<kQ8_0> {
    uint32_t d;
    u128_a2 q0, q1;
    __device__ __forceinline__ void load(const uint8_t *p) {
        d = load_u16(p);
        q0 = *reinterpret_cast<const u128_a2 *>(p + 2);
        q1 = *reinterpret_cast<const u128_a2 *>(p + 18);
    }
    // int8 q = (q ^ 0x80) - 128 with the xor-ed byte read as unsigned.
    __device__ __forceinline__ float dot(const float *xv, float xsum) const {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t a = q0.v[w] ^ 0x80808080u, b = q1.v[w] ^ 0x80808080u;
            s0 = fmaf(ubyte0(a), xv[4 * w + 0], s0);
            s0 = fmaf(ubyte1(a), xv[4 * w + 1], s0);
            s0 = fmaf(ubyte2(a), xv[4 * w + 2], s0);
            s0 = fmaf(ubyte3(a), xv[4 * w + 3], s0);
            s1 = fmaf(ubyte0(b), xv[16 + 4 * w + 0], s1);
            s1 = fmaf(ubyte1(b), xv[16 + 4 * w + 1], s1);
            s1 = fmaf(ubyte2(b), xv[16 + 4 * w + 2], s1);
            s1 = fmaf(ubyte3(b), xv[16 + 4 * w + 3], s1);
        }
        return half_bits_to_float(d) * ((s0 + s1) - 128.0f * xsum);
    }
};

__device__ __forceinline__ float sum32(const float *v) {
    float a = 0.f, b = 0.f, c = 0.f, d = 0.f;
#pragma unroll
    for (int i = 0; i < 32; i += 4) { a += v[i]; b += v[i + 1]; c += v[i + 2]; d += v[i + 3]; }
    return (a + b) + (c + d);
}

__device__ __forceinline__ float4 load_x4(const float *x, int64_t i, bool aligned) {
    if (aligned) return reinterpret_cast<const float4 *>(x)[i];
    return make_float4(x[4 * i], x[4 * i + 1], x[4 * i + 2], x[4 * i + 3]);
}

// ---- 32-value block formats -----------------------------------------------------------
//
// LDS layout of the activation chunk: float4 #j (0..7) of block b lives at xs[j * nbc + b],
// so the 64 lanes (consecutive b) of a ds_read_b128 touch consecutive 16-byte slots.
template <int T, int R, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv_b32_kernel(const float *__restrict__ X, const uint8_t *__restrict__ W,
                                                              const float *__restrict__ bias, float *__restrict__ Y,
                                                              int K, int N, int64_t row_bytes, int kchunk, int act) {
    extern __shared__ float4 xs[];
    constexpr int bpb = Geom<T>::bpb;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *x = X + (int64_t)blockIdx.y * K;
    float *y = Y + (int64_t)blockIdx.y * N;
    const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    const int ngroups = (N + R - 1) / R;
    const int grp = blockIdx.x * WAVES + wave;  // one group of R rows per wavefront
    const int row0 = grp * R;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;

    for (int k0 = 0; k0 < K; k0 += kchunk) {
        const int kc = min(kchunk, K - k0);
        const int nbc = kc >> 5;
        if (k0 > 0) __syncthreads();
        for (int i = tid; i < (kc >> 2); i += WAVES * 64) xs[(i & 7) * nbc + (i >> 3)] = load_x4(x + k0, i, aligned);
        __syncthreads();
        if (grp < ngroups) {
            for (int b0 = 0; b0 < nbc; b0 += 64) {
                const int b = b0 + lane;
                if (b < nbc) {
                    LaneBlock<T> blk[R];
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const int row = min(row0 + r, N - 1);
                        blk[r].load(W + (int64_t)row * row_bytes + (int64_t)((k0 >> 5) + b) * bpb);
                    }
                    float xv[32];
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const float4 t = xs[j * nbc + b];
                        xv[4 * j] = t.x; xv[4 * j + 1] = t.y; xv[4 * j + 2] = t.z; xv[4 * j + 3] = t.w;
                    }
                    const float xsum = sum32(xv);
#pragma unroll
                    for (int r = 0; r < R; r++) acc[r] += blk[r].dot(xv, xsum);
                }
            }
        }
    }
    if (grp >= ngroups) return;
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = wave_sum(acc[r]);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = row0 + r;
            if (row < N) y[row] = apply_act(act, acc[r] + (bias ? bias[row] : 0.f));
        }
    }
}

// ---- 32-value block formats, two blocks per lane ---------------------------------------
//
// The fast path whenever K is a multiple of 64.  A pair of consecutive blocks (36 bytes for
// Q4_0 / IQ4_NL, 68 bytes for Q8_0) starts on a 4-byte boundary, so a lane fetches its pair
// as whole dwords (dwordx4 ... + dword) and realigns the first block's payload in registers
// with v_alignbit.  Measured on MI355X this pattern streams as fast as perfectly aligned
// 16-byte loads, while one 18-byte block per lane (2-byte aligned loads) costs ~30 %.
// The weight loads of the first step are issued before the activations are staged, so the
// HBM latency overlaps the LDS fill and its barrier.
template <int T> struct LanePair;

template <> struct LanePair<kQ4_0> {
    struct __attribute__((packed, aligned(4))) Raw { uint32_t v[9]; };
    Raw raw;
    __device__ __forceinline__ void load(const uint8_t *p) { raw = *reinterpret_cast<const Raw *>(p); }
    __device__ __forceinline__ float dot(const float *xv, float xsum0, float xsum1) const {
        const uint32_t *v = raw.v;
        float r0, r1;
        {
            float lo = 0.f, hi = 0.f;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t q = __builtin_amdgcn_alignbit(v[w + 1], v[w], 16);
                const uint32_t l = q & 0x0F0F0F0Fu, h = q & 0xF0F0F0F0u;
                lo = fmaf(ubyte0(l), xv[4 * w + 0], lo);
                lo = fmaf(ubyte1(l), xv[4 * w + 1], lo);
                lo = fmaf(ubyte2(l), xv[4 * w + 2], lo);
                lo = fmaf(ubyte3(l), xv[4 * w + 3], lo);
                hi = fmaf(ubyte0(h), xv[16 + 4 * w + 0], hi);
                hi = fmaf(ubyte1(h), xv[16 + 4 * w + 1], hi);
                hi = fmaf(ubyte2(h), xv[16 + 4 * w + 2], hi);
                hi = fmaf(ubyte3(h), xv[16 + 4 * w + 3], hi);
            }
            r0 = half_bits_to_float(v[0] & 0xFFFFu) * (fmaf(hi, 0.0625f, lo) - 8.0f * xsum0);
        }
        {
            float lo = 0.f, hi = 0.f;
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t q = v[5 + w];
                const uint32_t l = q & 0x0F0F0F0Fu, h = q & 0xF0F0F0F0u;
                lo = fmaf(ubyte0(l), xv[32 + 4 * w + 0], lo);
                lo = fmaf(ubyte1(l), xv[32 + 4 * w + 1], lo);
                lo = fmaf(ubyte2(l), xv[32 + 4 * w + 2], lo);
                lo = fmaf(ubyte3(l), xv[32 + 4 * w + 3], lo);
                hi = fmaf(ubyte0(h), xv[48 + 4 * w + 0], hi);
                hi = fmaf(ubyte1(h), xv[48 + 4 * w + 1], hi);
                hi = fmaf(ubyte2(h), xv[48 + 4 * w + 2], hi);
                hi = fmaf(ubyte3(h), xv[48 + 4 * w + 3], hi);
            }
            r1 = half_bits_to_float(v[4] >> 16) * (fmaf(hi, 0.0625f, lo) - 8.0f * xsum1);
        }
        return r0 + r1;
    }
};

template <> struct LanePair<kIQ4_NL> {
    struct __attribute__((packed, aligned(4))) Raw { uint32_t v[9]; };
    Raw raw;
    __device__ __forceinline__ void load(const uint8_t *p) { raw = *reinterpret_cast<const Raw *>(p); }
    __device__ __forceinline__ float dot(const float *xv, float, float) const {
        const uint32_t *v = raw.v;
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t qa = __builtin_amdgcn_alignbit(v[w + 1], v[w], 16), qb = v[5 + w];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t a = (qa >> (8 * j)) & 0xFFu, b = (qb >> (8 * j)) & 0xFFu;
                s0 = fmaf(iq4nl_value(a & 15u), xv[4 * w + j], s0);
                s0 = fmaf(iq4nl_value(a >> 4), xv[16 + 4 * w + j], s0);
                s1 = fmaf(iq4nl_value(b & 15u), xv[32 + 4 * w + j], s1);
                s1 = fmaf(iq4nl_value(b >> 4), xv[48 + 4 * w + j], s1);
            }
        }
        return half_bits_to_float(v[0] & 0xFFFFu) * s0 + half_bits_to_float(v[4] >> 16) * s1;
    }
};

template <> struct LanePair<kQ8_0> {
    struct __attribute__((packed, aligned(4))) Raw { uint32_t v[17]; };
    Raw raw;
    __device__ __forceinline__ void load(const uint8_t *p) { raw = *reinterpret_cast<const Raw *>(p); }
    __device__ __forceinline__ float dot(const float *xv, float xsum0, float xsum1) const {
        const uint32_t *v = raw.v;
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < 8; w++) {
            const uint32_t a = __builtin_amdgcn_alignbit(v[w + 1], v[w], 16) ^ 0x80808080u;
            const uint32_t b = v[9 + w] ^ 0x80808080u;
            s0 = fmaf(ubyte0(a), xv[4 * w + 0], s0);
            s0 = fmaf(ubyte1(a), xv[4 * w + 1], s0);
            s0 = fmaf(ubyte2(a), xv[4 * w + 2], s0);
            s0 = fmaf(ubyte3(a), xv[4 * w + 3], s0);
            s1 = fmaf(ubyte0(b), xv[32 + 4 * w + 0], s1);
            s1 = fmaf(ubyte1(b), xv[32 + 4 * w + 1], s1);
            s1 = fmaf(ubyte2(b), xv[32 + 4 * w + 2], s1);
            s1 = fmaf(ubyte3(b), xv[32 + 4 * w + 3], s1);
        }
        return half_bits_to_float(v[0] & 0xFFFFu) * (s0 - 128.0f * xsum0) +
               half_bits_to_float(v[8] >> 16) * (s1 - 128.0f * xsum1);
    }
};

// LDS layout of the activation chunk: float4 #j (0..15) of pair p lives at xs[j * npc + p].
template <int T, int R, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv_pair_kernel(const float *__restrict__ X, const uint8_t *__restrict__ W,
                                                               const float *__restrict__ bias, float *__restrict__ Y,
                                                               int K, int N, int64_t row_bytes, int kchunk, int act) {
    extern __shared__ float4 xs[];
    constexpr int pair_bytes = 2 * Geom<T>::bpb;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *x = X + (int64_t)blockIdx.y * K;
    float *y = Y + (int64_t)blockIdx.y * N;
    const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    const int ngroups = (N + R - 1) / R;
    const int grp = blockIdx.x * WAVES + wave;
    const bool live = grp < ngroups;
    const int row0 = grp * R;
    const uint8_t *wrow[R];
#pragma unroll
    for (int r = 0; r < R; r++) wrow[r] = W + (int64_t)min(row0 + r, N - 1) * row_bytes;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;

    LanePair<T> cur[R];
    const int np_total = K >> 6;
    if (live && lane < np_total) {
#pragma unroll
        for (int r = 0; r < R; r++) cur[r].load(wrow[r] + (int64_t)lane * pair_bytes);
    }
    for (int k0 = 0; k0 < K; k0 += kchunk) {
        const int kc = min(kchunk, K - k0);
        const int npc = kc >> 6;
        if (k0 > 0) __syncthreads();
        for (int i = tid; i < (kc >> 2); i += WAVES * 64) xs[(i & 15) * npc + (i >> 4)] = load_x4(x + k0, i, aligned);
        __syncthreads();
        if (!live) continue;
        for (int p0 = 0; p0 < npc; p0 += 64) {
            const int p = p0 + lane;
            // prefetch the next step's pairs (next 64 pairs of the row, possibly in the next chunk)
            LanePair<T> nxt[R];
            const int pn = (k0 >> 6) + p0 + 64 + lane;
            const bool more = pn < np_total;
            if (more) {
#pragma unroll
                for (int r = 0; r < R; r++) nxt[r].load(wrow[r] + (int64_t)pn * pair_bytes);
            }
            if (p < npc) {
                float xv[64];
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    const float4 t = xs[j * npc + p];
                    xv[4 * j] = t.x; xv[4 * j + 1] = t.y; xv[4 * j + 2] = t.z; xv[4 * j + 3] = t.w;
                }
                const float xsum0 = sum32(xv), xsum1 = sum32(xv + 32);
#pragma unroll
                for (int r = 0; r < R; r++) acc[r] += cur[r].dot(xv, xsum0, xsum1);
            }
            if (more) {
#pragma unroll
                for (int r = 0; r < R; r++) cur[r] = nxt[r];
            }
        }
    }
    if (!live) return;
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = wave_sum(acc[r]);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = row0 + r;
            if (row < N) y[row] = apply_act(act, acc[r] + (bias ? bias[row] : 0.f));
        }
    }
}

// ---- Q4_K -----------------------------------------------------------------------------
//
// Eight lanes share one 144-byte super-block: lane part i (0..7) takes code bytes
// 16i..16i+15, i.e. group g = i/2 and half p = i%2; the low nibbles are 16 values of
// sub-block 2g, the high nibbles 16 values of sub-block 2g+1.  All eight lanes read the
// same 16-byte header (d, dmin, packed scales) - one broadcast load.
// LDS layout: unit u = 8*sb + i holds its 8 float4 of x (4 for the low-nibble run, 4 for
// the high-nibble run) at xs[j * nunits + u].
template <int R, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv_q4k_kernel(const float *__restrict__ X, const uint8_t *__restrict__ W,
                                                              const float *__restrict__ bias, float *__restrict__ Y,
                                                              int K, int N, int64_t row_bytes, int kchunk, int act) {
    extern __shared__ float4 xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *x = X + (int64_t)blockIdx.y * K;
    float *y = Y + (int64_t)blockIdx.y * N;
    const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    const int ngroups = (N + R - 1) / R;
    const int grp = blockIdx.x * WAVES + wave;
    const int row0 = grp * R;
    const int part = lane & 7, sbl = lane >> 3, g = part >> 1;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;

    for (int k0 = 0; k0 < K; k0 += kchunk) {
        const int kc = min(kchunk, K - k0);
        const int nunits = kc >> 5, nsb = kc >> 8;
        if (k0 > 0) __syncthreads();
        for (int f = tid; f < (kc >> 2); f += WAVES * 64) {
            const int sb = f >> 6, r = f & 63, rr = r & 15;
            const int unit = sb * 8 + (r >> 4) * 2 + ((rr >> 2) & 1);
            const int j = (rr >> 3) * 4 + (rr & 3);
            xs[j * nunits + unit] = load_x4(x + k0, f, aligned);
        }
        __syncthreads();
        if (grp < ngroups) {
            for (int s0 = 0; s0 < nsb; s0 += 8) {
                const int sb = s0 + sbl;
                if (sb < nsb) {
                    uint4 hd[R], q[R];
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const int row = min(row0 + r, N - 1);
                        const uint8_t *p = W + (int64_t)row * row_bytes + (int64_t)((k0 >> 8) + sb) * 144;
                        hd[r] = *reinterpret_cast<const uint4 *>(p);
                        q[r] = *reinterpret_cast<const uint4 *>(p + 16 + 16 * part);
                    }
                    float xv[32];
                    const int unit = sb * 8 + part;
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const float4 t = xs[j * nunits + unit];
                        xv[4 * j] = t.x; xv[4 * j + 1] = t.y; xv[4 * j + 2] = t.z; xv[4 * j + 3] = t.w;
                    }
                    float sum_lo = 0.f, sum_hi = 0.f;
#pragma unroll
                    for (int i = 0; i < 16; i++) { sum_lo += xv[i]; sum_hi += xv[16 + i]; }
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const uint32_t qq[4] = {q[r].x, q[r].y, q[r].z, q[r].w};
                        float lo = 0.f, hi = 0.f;
#pragma unroll
                        for (int w = 0; w < 4; w++) {
                            const uint32_t l = qq[w] & 0x0F0F0F0Fu, h = qq[w] & 0xF0F0F0F0u;
                            lo = fmaf(ubyte0(l), xv[4 * w + 0], lo);
                            lo = fmaf(ubyte1(l), xv[4 * w + 1], lo);
                            lo = fmaf(ubyte2(l), xv[4 * w + 2], lo);
                            lo = fmaf(ubyte3(l), xv[4 * w + 3], lo);
                            hi = fmaf(ubyte0(h), xv[16 + 4 * w + 0], hi);
                            hi = fmaf(ubyte1(h), xv[16 + 4 * w + 1], hi);
                            hi = fmaf(ubyte2(h), xv[16 + 4 * w + 2], hi);
                            hi = fmaf(ubyte3(h), xv[16 + 4 * w + 3], hi);
                        }
                        uint32_t sc0, m0, sc1, m1;
                        q4k_scale_min(hd[r].y, hd[r].z, hd[r].w, 2 * g, sc0, m0);
                        q4k_scale_min(hd[r].y, hd[r].z, hd[r].w, 2 * g + 1, sc1, m1);
                        const float d = half_bits_to_float(hd[r].x & 0xFFFFu);
                        const float dmin = half_bits_to_float(hd[r].x >> 16);
                        const float pos = fmaf((float)sc1 * 0.0625f, hi, (float)sc0 * lo);
                        const float neg = fmaf((float)m1, sum_hi, (float)m0 * sum_lo);
                        acc[r] += d * pos - dmin * neg;
                    }
                }
            }
        }
    }
    if (grp >= ngroups) return;
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = wave_sum(acc[r]);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = row0 + r;
            if (row < N) y[row] = apply_act(act, acc[r] + (bias ? bias[row] : 0.f));
        }
    }
}

// ---- formats that only provide the 16-value decoder (Q6_K): one wavefront per row, lanes stride
// over the runs of 16 weights, activations straight from global memory (they stay in L2).
template <int T, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv_run16_kernel(const float *__restrict__ X, const uint8_t *__restrict__ W,
                                                                const float *__restrict__ bias, float *__restrict__ Y, int K, int N,
                                                                int64_t row_bytes, int act, int x_aligned) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = blockIdx.x * WAVES + wave;
    if (row >= N) return;
    const float *x = X + (int64_t)blockIdx.y * K;
    const uint8_t *wrow = W + (int64_t)row * row_bytes;
    const int runs = K >> 4;
    float acc = 0.f;
    for (int i = lane; i < runs; i += 64) {
        float w[16], xv[16];
        dequant16<T>(wrow, i, w);
        if (x_aligned) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float4 t = reinterpret_cast<const float4 *>(x)[4 * i + j];
                xv[4 * j] = t.x; xv[4 * j + 1] = t.y; xv[4 * j + 2] = t.z; xv[4 * j + 3] = t.w;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; j++) xv[j] = x[16 * i + j];
        }
#pragma unroll
        for (int j = 0; j < 16; j++) acc = fmaf(w[j], xv[j], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) Y[(int64_t)blockIdx.y * N + row] = apply_act(act, acc + (bias ? bias[row] : 0.f));
}

template <int T>
int launch_run16(const float *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
                 hipStream_t s) {
    constexpr int WAVES = 4;
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    const dim3 grid((unsigned)((N + WAVES - 1) / WAVES), (unsigned)M);
    const int aligned = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (K % 4) == 0;
    return launch(gemv_run16_kernel<T, WAVES>, grid, dim3(WAVES * 64), 0, s, x, W, bias, y, (int)K, (int)N, row_bytes, act, aligned);
}

// ---- host side --------------------------------------------------------------------------

// Two rows per wavefront, eight wavefronts per workgroup (the best of the combinations measured).
constexpr int kRowsPerWave = 2, kWavesPerWG = 8;

constexpr int kMaxChunk = 16384;  // fp32 activations staged in LDS per pass: 64 KiB

template <int T, int R, int WAVES>
int launch_one(const float *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
               hipStream_t s) {
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    const int kchunk = (int)(K < kMaxChunk ? K : kMaxChunk);
    const size_t shmem = (size_t)kchunk * sizeof(float);
    const int64_t ngroups = (N + R - 1) / R;
    const dim3 grid((unsigned)((ngroups + WAVES - 1) / WAVES), (unsigned)M);
    if constexpr (T == kQ4_K) {
        return launch(gemv_q4k_kernel<R, WAVES>, grid, dim3(WAVES * 64), shmem, s, x, W, bias, y, (int)K, (int)N,
                      row_bytes, kchunk, act);
    } else {
        if (K % 64 == 0)
            return launch(gemv_pair_kernel<T, R, WAVES>, grid, dim3(WAVES * 64), shmem, s, x, W, bias, y, (int)K, (int)N,
                          row_bytes, kchunk, act);
        return launch(gemv_b32_kernel<T, R, WAVES>, grid, dim3(WAVES * 64), shmem, s, x, W, bias, y, (int)K, (int)N,
                      row_bytes, kchunk, act);
    }
}

template <int T>
int launch_type(const float *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias, int act, float *y,
                hipStream_t s) {
    return launch_one<T, kRowsPerWave, kWavesPerWG>(x, M, K, W, N, bias, act, y, s);
}

}  // namespace

int launch_gemv(int type, const float *x, int64_t M, int64_t K, const uint8_t *W, int64_t N, const float *bias,
                int act, float *y, hipStream_t s) {
    if (M == 0 || N == 0) return GQ_OK;
    if (N > INT32_MAX || K > INT32_MAX || M > 65535)
        return fail(GQ_ERR_NOT_IMPLEMENTED, "gemv: dimensions M=%lld K=%lld N=%lld exceed the kernel's index range",
                    (long long)M, (long long)K, (long long)N);
    switch (type) {
    case kQ4_0: return launch_type<kQ4_0>(x, M, K, W, N, bias, act, y, s);
    case kQ8_0: return launch_type<kQ8_0>(x, M, K, W, N, bias, act, y, s);
    case kIQ4_NL: return launch_type<kIQ4_NL>(x, M, K, W, N, bias, act, y, s);
    case kQ4_K: return launch_type<kQ4_K>(x, M, K, W, N, bias, act, y, s);
    case kQ6_K: return launch_run16<kQ6_K>(x, M, K, W, N, bias, act, y, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "qdense: ggml type %d is not implemented", type);
    }
}

}  // namespace gq
