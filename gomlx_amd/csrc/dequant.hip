// ggml.Dequantize (ml/ggml/dequant.go:39-54) and ggml.EmbeddingLookupDecomposed
// (ml/ggml/gather.go:21-49) as gfx950 kernels.  Both are bit-exact with the reference
// arithmetic and bound by the fp32 writes (4 bytes out per 0.56-1.06 bytes in).
#include "blocks.hpp"
#include "common.hpp"

namespace gq {

// One thread produces 16 consecutive fp32 values (64 contiguous bytes) of one row; the 64
// lanes of a wavefront therefore write 4 KiB of contiguous output per row segment.
template <int T>
__global__ __launch_bounds__(256) void dequant_rows_kernel(const uint8_t *__restrict__ W, float *__restrict__ out,
                                                           int64_t N, int64_t K, int64_t row_bytes,
                                                           const int32_t *__restrict__ indices, int64_t vocab,
                                                           int32_t *__restrict__ err_flag) {
    const int64_t runs_per_row = K >> 4;
    const int64_t total = N * runs_per_row;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total;
         t += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = t / runs_per_row;
        const int64_t i = t - r * runs_per_row;
        int64_t src = r;
        bool bad = false;
        if (indices != nullptr) {  // gather: row r of the output is row indices[r] of the table
            src = indices[r];
            bad = src < 0 || src >= vocab;
            if (bad) src = 0;
        }
        float v[16];
        dequant16<T>(W + src * row_bytes, i, v);
        if (bad) {
            if (i == 0 && err_flag != nullptr) *err_flag = 1;
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = __builtin_nanf("");
        }
        float4 *o = reinterpret_cast<float4 *>(out + r * K + i * 16);
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = make_float4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]);
    }
}

template <int T>
static int launch_rows(const uint8_t *W, float *out, int64_t N, int64_t K, const int32_t *indices, int64_t vocab,
                       int32_t *err_flag, hipStream_t s) {
    const int64_t row_bytes = (K / Geom<T>::vpb) * Geom<T>::bpb;
    const int64_t total = N * (K >> 4);
    if (total == 0) return GQ_OK;
    const int64_t want = (total + 255) / 256;
    const int64_t cap = (int64_t)device_cu_count() * 32;  // grid-stride beyond 8 blocks per SIMD
    const unsigned grid = (unsigned)(want < cap ? want : cap);
    return launch(dequant_rows_kernel<T>, dim3(grid), dim3(256), 0, s, W, out, N, K, row_bytes, indices, vocab,
                  err_flag);
}

static int dispatch_rows(int type, const uint8_t *W, float *out, int64_t N, int64_t K, const int32_t *indices,
                         int64_t vocab, int32_t *err_flag, hipStream_t s) {
    switch (type) {
    case kQ8_0: return launch_rows<kQ8_0>(W, out, N, K, indices, vocab, err_flag, s);
    case kQ4_0: return launch_rows<kQ4_0>(W, out, N, K, indices, vocab, err_flag, s);
    case kIQ4_NL: return launch_rows<kIQ4_NL>(W, out, N, K, indices, vocab, err_flag, s);
    case kQ4_K: return launch_rows<kQ4_K>(W, out, N, K, indices, vocab, err_flag, s);
    case kQ6_K: return launch_rows<kQ6_K>(W, out, N, K, indices, vocab, err_flag, s);
    default: return fail(GQ_ERR_NOT_IMPLEMENTED, "dequantize: ggml type %d is not implemented", type);
    }
}

int launch_dequantize(int type, const uint8_t *W, int64_t N, int64_t K, float *out, hipStream_t s) {
    return dispatch_rows(type, W, out, N, K, nullptr, 0, nullptr, s);
}

int launch_embedding_lookup(int type, const uint8_t *table, int64_t vocab, int64_t K, const int32_t *idx,
                            int64_t count, float *out, int32_t *err_flag, hipStream_t s) {
    return dispatch_rows(type, table, out, count, K, idx, vocab, err_flag, s);
}

}  // namespace gq
