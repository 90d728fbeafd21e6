// C ABI of libgomlx_hipq.so: argument validation, device selection, dispatch to the kernel
// families, HIP-graph recording and per-kernel timing.  See include/gomlx_hipq.h for the
// contract of every entry point and the reference interface it replaces.
#include "common.hpp"
#include "workspace.hpp"

#include <atomic>
#include <cstring>
#include <cstdlib>
#include <map>
#include <mutex>
#include <new>

namespace gq {

namespace {
thread_local char g_error[512] = "";
std::atomic<int> g_device{-1};
std::atomic<int> g_cu_count{256};
std::mutex g_init_mutex;
}  // namespace

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return status;
}

int hip_fail(hipError_t e, const char *what) {
    if (e == hipErrorOutOfMemory) return fail(GQ_ERR_OOM, "%s: %s", what, hipGetErrorString(e));
    if (e == hipErrorNoDevice || e == hipErrorInvalidDevice)
        return fail(GQ_ERR_NO_DEVICE, "%s: %s", what, hipGetErrorString(e));
    return fail(GQ_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

int use_device() {
    const int dev = g_device.load(std::memory_order_acquire);
    if (dev < 0) return fail(GQ_ERR_NO_DEVICE, "gq_init() has not been called (or failed)");
    int cur = -1;
    if (hipGetDevice(&cur) != hipSuccess || cur != dev) GQ_HIP(hipSetDevice(dev));
    return GQ_OK;
}

int device_cu_count() { return g_cu_count.load(std::memory_order_relaxed); }

// ---- scratch memory ------------------------------------------------------------------------------
// Per-stream buffers come from the pool of workspace.hpp (sequence lock per stream, buffers pinned by
// recorded graphs, released with their stream).  A call through gq_qdense_f32_static is served from
// the fixed device array below instead and never allocates.
namespace {

constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
constexpr int kMaxDevices = 64;
// Scratch of the entry point that allocates nothing.  Host code never uses this name as an address:
// g_scratch_ptr[device] holds the array's device address, taken once in gq_init().
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
void *g_scratch_ptr[kMaxDevices] = {};

int ws_alloc(void **p, size_t bytes) {
    GQ_HIP(hipMalloc(p, bytes));
    // the flag words at the head of a buffer start at zero (allocation never happens inside a recording)
    hipError_t e = hipMemsetAsync(*p, 0, bytes < kWsSyncBytes ? bytes : kWsSyncBytes, nullptr);
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    if (e != hipSuccess) { (void)hipFree(*p); *p = nullptr; return hip_fail(e, "hipMemsetAsync(workspace flags)"); }
    return GQ_OK;
}
void ws_release(void *p) { (void)hipFree(p); }
void ws_sync(const void *s) { (void)hipStreamSynchronize((hipStream_t)const_cast<void *>(s)); }
bool ws_capturing(const void *s) {
    if (!s) return false;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing((hipStream_t)const_cast<void *>(s), &st) == hipSuccess && st != hipStreamCaptureStatusNone;
}
WorkspacePool &pool() {
    static WorkspacePool *p = new WorkspacePool(WsHooks{ws_alloc, ws_release, ws_sync, ws_capturing});  // never destroyed: outlives every caller
    return *p;
}

// One per ABI call that may reach a path with scratch memory; nested calls share the outermost one.
struct RecordedGraph {  // what gq_graph_end hands out
    hipGraphExec_t exec;
    hipStream_t stream;               // the stream it was recorded on, the only one it replays on
    std::vector<WsBlockRef> blocks;   // workspaces its launches point at
};

struct CallScope;
thread_local CallScope *t_scope = nullptr;
struct CallScope {
    SeqLock lock;
    unsigned char *static_ptr = nullptr;  // set: requests are served from the static array
    bool outer;
    CallScope() : outer(t_scope == nullptr) { if (outer) t_scope = this; }
    ~CallScope() { if (outer) t_scope = nullptr; }
};

}  // namespace

int stream_workspace(hipStream_t s, size_t bytes, void **out, int slot, uint32_t **sync) {
    CallScope *sc = t_scope;
    if (!sc) return fail(GQ_ERR_INVALID, "internal: scratch memory requested outside an entry point");
    void *base = nullptr;
    if (sc->static_ptr) {
        // (the static array is zero when the library is loaded: its first kWsSyncBytes are the flag words)
        if (slot != 0 || bytes > kStaticScratchBytes - kWsSyncBytes)
            return fail(GQ_ERR_INVALID, "gq_qdense_f32_static: this call needs %zu bytes of scratch memory, the static buffer holds %zu; use gq_qdense_f32",
                        bytes, kStaticScratchBytes - kWsSyncBytes);
        base = sc->static_ptr;
    } else {
        if (slot < 0 || slot >= kWsSlots) return fail(GQ_ERR_INVALID, "internal: workspace slot %d", slot);
        if (!sc->lock.held()) sc->lock.lock(pool().stream(s));
        const int rc = pool().acquire(*sc->lock.held(), s, slot, bytes + kWsSyncBytes, &base);
        if (rc == kWsWouldAllocateInRecording)
            return fail(GQ_ERR_INVALID, "qdense: the %zu-byte workspace of this stream must exist before a graph is recorded; run the "
                        "same call once outside the recording first", bytes);
        if (rc) return rc;
    }
    *out = static_cast<unsigned char *>(base) + kWsSyncBytes;
    if (sync) *sync = static_cast<uint32_t *>(base);
    return GQ_OK;
}

ProfileState &profile_state() {
    thread_local ProfileState ps;
    return ps;
}

namespace {

struct TypeInfo { int bpb, vpb; };

bool type_info(int type, TypeInfo &ti) {
    switch (type) {
    case GQ_Q4_0: ti = {18, 32}; return true;
    case GQ_Q8_0: ti = {34, 32}; return true;
    case GQ_Q4_K: ti = {144, 256}; return true;
    case GQ_Q6_K: ti = {210, 256}; return true;
    case GQ_IQ4_NL: ti = {18, 32}; return true;
    default: return false;
    }
}

constexpr int64_t kGemvMaxRows = 16;  // above this many activation rows the tiled MFMA kernels win
// Batched submissions merge problems of up to this many activation rows each into one K-sliced GEMV launch (q/k/v
// of a decoder layer behind one normalisation, 2 / 4 / 8 rows: the layer's four calls take 50.6 / 83.1 / 86.8 us
// merged against 59.1 / 97.6 / 97.7 us as three calls).
// Only matrices under 24 MB are merged at several rows: over larger ones a single call serves several rows per pass.
int64_t batch_rows_max() { return 8; }

bool aligned_to(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Run-time argument checks shared by the dense entry points.
int check_dense_args(const char *fn, int type, const void *x, int64_t M, int64_t K, const void *W, int64_t N,
                     const float *bias, int act, const float *y, size_t x_align) {
    TypeInfo ti;
    if (!type_info(type, ti)) return fail(GQ_ERR_NOT_IMPLEMENTED, "%s: ggml type %d is not implemented", fn, type);
    if (M < 0 || N < 0) return fail(GQ_ERR_INVALID, "%s: negative dimension (M=%lld, N=%lld)", fn, (long long)M, (long long)N);
    if (K <= 0 || K % ti.vpb != 0)
        return fail(GQ_ERR_INVALID, "%s: K=%lld is not a positive multiple of the block size %d", fn, (long long)K, ti.vpb);
    if (act < GQ_ACT_NONE || act > GQ_ACT_TANH) return fail(GQ_ERR_INVALID, "%s: unknown activation %d", fn, act);
    if (M == 0 || N == 0) return GQ_OK;
    if (!x || !W || !y) return fail(GQ_ERR_INVALID, "%s: null device pointer", fn);
    if (!aligned_to(x, x_align)) return fail(GQ_ERR_INVALID, "%s: x must be %zu-byte aligned", fn, x_align);
    if (!aligned_to(W, 16)) return fail(GQ_ERR_INVALID, "%s: weights must be 16-byte aligned", fn);
    if (!aligned_to(y, 4) || (bias && !aligned_to(bias, 4))) return fail(GQ_ERR_INVALID, "%s: y / bias must be 4-byte aligned", fn);
    return GQ_OK;
}

// Batch sizes served by the split-K small-batch kernels: measured crossovers against the GEMV passes
// below and the two-pass GEMM above.  GEMV passes cost time in proportion to the weight bytes (small
// matrices: a pass per row, sharing W through the caches; large ones: a pass per four rows, two for
// Q6_K), the split-K kernels a fixed part plus less per byte.
// Measured (us per call in a replayed graph of dependent calls; rows 4 5 6 7 8 9 10; GEMV passes | split-K, flat over these rows):
//   Q8_0   4096x4096 (18 MB)  12.5 14.3 16.2 17.9 19.9 21.9 23.9 | 14.4   4096x14336 (62 MB) 17.3 27.2 28.0 30.2 27.7 37.9 38.9 | 29.3
//          4096x1024 (4 MB)    4.8  5.6  6.1  6.4  6.6  8.1  8.2 | 12.9   14336x4096         23.0 32.5 34.0 38.7 36.7 47.3 49.6 | 30.1
//   Q4_0   4096x4096 (9 MB)    9.6 10.7 12.0 13.5 15.1 16.5 18.0 | 13.0   4096x14336 (33 MB) 14.9 20.7 22.0 27.3 25.8 32.6 34.0 | 23.7
//          4096x1024 (2 MB)    4.2  4.8  4.8  5.5  5.6  6.2  6.3 | 12.1   14336x4096         19.4 25.2 28.1 34.8 33.0 40.1 43.2 | 24.7
//   Q4_K   4096x4096          11.1 12.6 14.6 16.6 18.6 20.5 22.5 | 13.1   4096x14336         15.8 22.3 24.1 29.1 27.5 34.9 36.8 | 19.3
//          4096x1024           4.4  5.4  6.2  6.4  6.5  7.4  8.0 | 12.3   14336x4096         20.4 26.9 29.8 36.7 35.0 42.7 46.0 | 19.6
//   Q6_K   4096x4096 (14 MB)  13.5 15.3 17.6 19.9 22.3 24.6 27.0 | 17.8   4096x14336 (48 MB) 25.6 34.6 34.6 44.2 44.3 54.0 54.2 | 33.0
//          4096x1024 (3 MB)    5.1  6.1  6.2  7.2  7.3  8.4  8.5 | 16.4   14336x4096         28.6 37.1 37.3 46.9 48.0 57.6 58.8 | 34.0
//   IQ4_NL 4096x4096          11.8 12.9 15.0 16.9 18.9 20.9 22.8 | 13.7   4096x14336         17.0 24.0 26.7 31.1 29.4 37.7 40.4 | 26.3
//          4096x1024           4.8  5.7  5.7  6.6  6.7  7.6  7.7 | 12.8   14336x4096         20.9 28.6 31.1 37.7 35.9 45.0 47.8 | 27.2
// The split-K route is three dependent launches with a floor of about 12 us: matrices of a few megabytes (the k / v
// projections of a grouped-query layer) stay on GEMV passes for every batch the GEMV takes.
// (The Q6_K kernel pays 16 scale groups per super-block: twice the time of the others per byte.)
constexpr int64_t kTinyWeightBytes = (int64_t)6 << 20;
int64_t split_k_from(int type, int64_t weight_bytes) {
    if (weight_bytes < kTinyWeightBytes) return kGemvMaxRows + 1;
    const bool large = weight_bytes >= kLargeWeightBytes;
    switch (type) {
    case GQ_Q8_0: return 6;
    case GQ_Q4_0: return large ? 6 : 7;
    case GQ_Q4_K: return large ? 5 : 6;
    case GQ_Q6_K: return large ? 5 : 6;
    case GQ_IQ4_NL: return 6;
    default: return 8;
    }
}
int64_t weight_bytes_of(int type, int64_t K, int64_t N) { return (int64_t)gq_row_bytes(type, K) * N; }
// Last batch size of the split-K kernels before the two-pass GEMM takes over.  The split-K route streams W once per 32
// batch rows; the two passes pay the 16-bit image (written once and read once, in proportion to N K) and a GEMM that splits
// K itself while its tiles are fewer than the CUs.
// Measured (python -m gomlx_amd.tune.crossover with GOMLX_HIPQ_SPLIT_K_TO=100000 and =16: us per call in a replayed graph of 20
// calls on rotating weights, fp32 activations; rows 32 64 96 128 160 192; split-K | two passes at the same rows):
//   Q8_0   4096x4096  16 22 27 29 35 36 | 27 28 29 30 31 31    4096x14336  32 37  43  49  69  76 | 56 56 55 58 69 69    14336x4096  32 38 44 49  70  77 | 63 70 72 73 81 82
//   Q4_0   4096x4096  15 20 25 26 32 33 | 25 26 26 27 29 29    4096x14336  27 33  40  45  61  67 | 57 55 55 56 67 69    14336x4096  28 34 40 45  62  69 | 62 63 69 68 79 79
//   Q4_K   4096x4096  15 17 21 29 36 38 | 26 26 27 29 30 30    4096x14336  25 28  34  38  53  57 | 61 59 60 60 73 72    14336x4096  21 30 36 41  55  59 | 69 73 72 71 85 85
//          (at 256 320 384 rows: 4096x14336 74 96 108 | 74 94 95; 14336x4096 77 99 112 | 87 108 109.  Q4_K walks up to four tiles of 32 batch rows per
//          launch; with one launch per 32 rows, as the other formats' kernels still work, it took 14 23 32 39 46 52, 27 44 61 79 96 113 and 22 36 49 63 77 92)
//   Q6_K   4096x4096  19 22 30 32 39 40 | 26 28 29 30 31 32    4096x14336  36 56  76  89 109 130 | 61 57 58 59 70 71    14336x4096  36 56 77 90 111 132 | 68 68 74 74 82 83
//   IQ4_NL 4096x4096  16 21 28 29 37 37 | 27 28 29 30 31 32    4096x14336  30 36  43  48  66  72 | 63 62 62 64 76 77    14336x4096  31 37 43 48  67  74 | 70 75 78 78 87 88
//          (Q8_0, Q4_0 and IQ4_NL walk up to four tiles of 32 batch rows per launch on the large matrices, like Q4_K; one pass per 32 rows took
//          33 52 71 84 100 118 / 33 52 72 85 104 121, 27 42 56 66 80 94 / 28 43 57 68 83 97 and 30 48 65 78 95 112 / 31 49 66 80 97 114; at 256
//          rows the tiles take 79 - 90 against 70 - 90)
// (Before the GEMM split K on narrow problems the two passes took 33 us on 4096x4096 and 92 .. 102 us on 14336x4096 at these rows.)
// GOMLX_HIPQ_SPLIT_K_TO=rows overrides the table (tuning runs only).
int64_t split_k_to_env() {
    static const int64_t v = [] { const char *e = std::getenv("GOMLX_HIPQ_SPLIT_K_TO"); return e ? (int64_t)std::atoll(e) : (int64_t)-1; }();
    return v;
}
int64_t split_k_to(int type, int64_t K, int64_t N) {
    if (split_k_to_env() >= 0) return split_k_to_env();
    const bool large = weight_bytes_of(type, K, N) >= kLargeWeightBytes, long_k = K > N;
    switch (type) {
    case GQ_Q8_0: return !large ? 128 : long_k ? 192 : 128;  // (4096x6144, 27 MB: 34 46 | 34 39 at 128 and 160 rows)
    case GQ_Q4_0: return !large ? 128 : 192;
    case GQ_Q4_K: return !large ? 128 : long_k ? 320 : 256;
    case GQ_Q6_K: return !large ? 96 : 64;
    case GQ_IQ4_NL: return !large ? 128 : 192;
    default: return 96;
    }
}

// The same point for a gated pair act(x.Wgate) * (x.Wup): both matrices are contracted against one activation image by the
// split-K kernels, or dequantised into one interleaved image for ONE GEMM by the two passes.  Measured (same tool, mode
// `gated`, SiLU; rows 32 64 96 128 160 192 256; split-K | two passes):
//   Q8_0   4096x4096  24 35 39 45 52 58 73 | 46 45 46 46 47 46 46    4096x14336  50 60  72  86 122 136 161 | 112 117 123 129 142 145 151
//   Q4_0   4096x4096  20 27 34 41 47 52 66 | 45 44 44 45 45 45 45    4096x14336  42 53  65  75 107 119 141 | 107 114 121 118 138 133 141
//   Q4_K   4096x4096  17 22 27 32 44 48 60 | 46 45 45 45 46 46 45    4096x14336  37 46  55  65  92 101 121 | 118 125 131 128 147 142 151
//          (one launch per 32 rows: 17 28 37 45 53 61 78 and 37 65 93 120 149 178 233; at 320 384 448 rows the large pair takes 173 198 243 | 203 205 209)
//   Q6_K   4096x4096  28 33 43 51 59 67 85 | 46 46 46 46 47 46 46    4096x14336  57 89 129 161 200 231 302 | 112 117 124 127 138 137 146
//   IQ4_NL 4096x4096  22 29 39 47 54 61 77 | 49 48 48 47 48 48 48    4096x14336  48 58  70  81 117 130 151 | 120 125 131 128 147 144 150
// (The pair composed of two dense calls and a multiplication is never ahead of the one GEMM: 127 - 159 against 118 - 143 us
// for Q4_K 4096 -> 2 x 14336 at 64 - 256 rows.)
int64_t gated_split_k_to(int type, int64_t K, int64_t N) {
    if (split_k_to_env() >= 0) return split_k_to_env();
    const bool large = weight_bytes_of(type, K, N) >= kLargeWeightBytes, long_k = K > N;
    if (large && long_k) return split_k_to(type, K, N);
    switch (type) {
    case GQ_Q8_0: return large ? 192 : 128;
    case GQ_Q4_0: return large ? 192 : 128;
    case GQ_Q4_K: return large ? 384 : 160;
    case GQ_Q6_K: return large ? 64 : 96;
    case GQ_IQ4_NL: return large ? 192 : 128;
    default: return 96;
    }
}

// large batches: W dequantised once into the stream's workspace, then a plain 16-bit GEMM
int two_pass(int type, bool x_is_bf16, const void *x, int64_t M, int64_t K, const void *W, int64_t N, const float *bias, int act,
             float *y, hipStream_t s) {
    void *ws = nullptr;
    if (int rc = stream_workspace(s, gemm_two_pass_workspace(x_is_bf16, M, K, N), &ws)) return rc;
    return launch_gemm_two_pass(type, x_is_bf16, x, M, K, static_cast<const uint8_t *>(W), N, bias, act, y, ws, s);
}

}  // namespace
}  // namespace gq

using namespace gq;

extern "C" {

int gq_abi_version(void) { return 1; }

int gq_bytes_per_block(int type) {
    TypeInfo ti;
    return type_info(type, ti) ? ti.bpb : 0;
}

int gq_values_per_block(int type) {
    TypeInfo ti;
    return type_info(type, ti) ? ti.vpb : 0;
}

size_t gq_row_bytes(int type, int64_t K) {
    TypeInfo ti;
    if (!type_info(type, ti) || K <= 0 || K % ti.vpb != 0) return 0;
    return (size_t)(K / ti.vpb) * (size_t)ti.bpb;
}

int gq_qdense_check(int type, int x_dtype, int64_t M, int64_t x_last_dim, int64_t N, int64_t w_row_bytes,
                    int64_t bias_len, int act, int64_t *K_out) {
    TypeInfo ti;
    if (!type_info(type, ti)) return fail(GQ_ERR_NOT_IMPLEMENTED, "FusedQuantizedDense: ggml type %d is not implemented", type);
    if (x_dtype != GQ_F32 && x_dtype != GQ_BF16)
        return fail(GQ_ERR_NOT_IMPLEMENTED, "FusedQuantizedDense: activation dtype %d is not implemented", x_dtype);
    if (M < 0 || N < 0) return fail(GQ_ERR_INVALID, "FusedQuantizedDense: negative dimension");
    if (w_row_bytes <= 0 || w_row_bytes % ti.bpb != 0)
        return fail(GQ_ERR_INVALID, "FusedQuantizedDense: weight row of %lld bytes is not a whole number of %d-byte blocks",
                    (long long)w_row_bytes, ti.bpb);
    const int64_t K = w_row_bytes / ti.bpb * ti.vpb;
    if (x_last_dim != K)  // ml/ggml/dense.go:38-41
        return fail(GQ_ERR_INVALID, "FusedQuantizedDense: x has %lld features but the weights decode to K=%lld",
                    (long long)x_last_dim, (long long)K);
    if (bias_len >= 0 && bias_len != N)
        return fail(GQ_ERR_INVALID, "FusedQuantizedDense: bias has %lld elements, expected N=%lld", (long long)bias_len, (long long)N);
    if (act < GQ_ACT_NONE || act > GQ_ACT_TANH) return fail(GQ_ERR_INVALID, "FusedQuantizedDense: unknown activation %d", act);
    if (K_out) *K_out = K;
    return GQ_OK;
}

int gq_device_count(int *count) {
    if (!count) return fail(GQ_ERR_INVALID, "gq_device_count: null argument");
    int n = 0;
    const hipError_t e = hipGetDeviceCount(&n);
    if (e == hipErrorNoDevice) { *count = 0; return GQ_OK; }
    if (e != hipSuccess) { *count = 0; return hip_fail(e, "hipGetDeviceCount"); }
    *count = n;
    return GQ_OK;
}

int gq_init(int device) {
    std::lock_guard<std::mutex> lock(g_init_mutex);
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) return fail(GQ_ERR_NO_DEVICE, "gq_init: no HIP device (%s)", hipGetErrorString(e));
    if (device < 0 || device >= n) return fail(GQ_ERR_NO_DEVICE, "gq_init: device %d out of range (found %d)", device, n);
    const int cur = g_device.load();
    if (cur >= 0 && cur != device)
        return fail(GQ_ERR_INVALID, "gq_init: already initialised on device %d (one device per process)", cur);
    hipDeviceProp_t prop;
    GQ_HIP(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(GQ_ERR_NO_DEVICE, "gq_init: device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
    GQ_HIP(hipSetDevice(device));
    if (device >= kMaxDevices) return fail(GQ_ERR_NO_DEVICE, "gq_init: device %d is beyond the %d this library keeps state for", device, kMaxDevices);
    if (!g_scratch_ptr[device]) {  // this device's copy of the static scratch array (each device has its own, at its own address)
        void *p = nullptr;
        GQ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        g_scratch_ptr[device] = p;
    }
    g_cu_count.store(prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256);
    g_device.store(device, std::memory_order_release);
    return GQ_OK;
}

int gq_device_name(char *buf, size_t n) {
    if (!buf || n == 0) return fail(GQ_ERR_INVALID, "gq_device_name: null buffer");
    if (int rc = use_device()) return rc;
    hipDeviceProp_t prop;
    GQ_HIP(hipGetDeviceProperties(&prop, g_device.load()));
    std::snprintf(buf, n, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
    return GQ_OK;
}

int gq_malloc(void **dptr, size_t bytes) {
    if (!dptr) return fail(GQ_ERR_INVALID, "gq_malloc: null argument");
    *dptr = nullptr;
    if (int rc = use_device()) return rc;
    if (bytes == 0) return GQ_OK;
    GQ_HIP(hipMalloc(dptr, bytes));
    return GQ_OK;
}

int gq_free(void *dptr) {
    if (!dptr) return GQ_OK;
    if (int rc = use_device()) return rc;
    GQ_HIP(hipFree(dptr));
    return GQ_OK;
}

int gq_h2d(void *d, const void *h, size_t bytes, void *stream) {
    if (bytes == 0) return GQ_OK;
    if (!d || !h) return fail(GQ_ERR_INVALID, "gq_h2d: null pointer");
    if (int rc = use_device()) return rc;
    GQ_HIP(hipMemcpyAsync(d, h, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    GQ_HIP(hipStreamSynchronize((hipStream_t)stream));
    return GQ_OK;
}

int gq_d2h(void *h, const void *d, size_t bytes, void *stream) {
    if (bytes == 0) return GQ_OK;
    if (!d || !h) return fail(GQ_ERR_INVALID, "gq_d2h: null pointer");
    if (int rc = use_device()) return rc;
    GQ_HIP(hipMemcpyAsync(h, d, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    GQ_HIP(hipStreamSynchronize((hipStream_t)stream));
    return GQ_OK;
}

int gq_stream_create(void **stream) {
    if (!stream) return fail(GQ_ERR_INVALID, "gq_stream_create: null argument");
    if (int rc = use_device()) return rc;
    hipStream_t s;
    GQ_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = s;
    return GQ_OK;
}

int gq_stream_destroy(void *stream) {
    if (!stream) return GQ_OK;
    if (int rc = use_device()) return rc;
    pool().destroy_stream(stream);  // waits for the stream, then frees its workspaces (those a recorded graph points at go with the graph)
    GQ_HIP(hipStreamDestroy((hipStream_t)stream));
    return GQ_OK;
}

int gq_sync(void *stream) {
    if (int rc = use_device()) return rc;
    GQ_HIP(hipStreamSynchronize((hipStream_t)stream));
    return GQ_OK;
}

int gq_dequantize(int type, const void *dW, int64_t N, int64_t K, float *dOut, void *stream) {
    TypeInfo ti;
    if (!type_info(type, ti)) return fail(GQ_ERR_NOT_IMPLEMENTED, "gq_dequantize: ggml type %d is not implemented", type);
    if (N < 0) return fail(GQ_ERR_INVALID, "gq_dequantize: negative N");
    if (K <= 0 || K % ti.vpb != 0)
        return fail(GQ_ERR_INVALID, "gq_dequantize: K=%lld is not a positive multiple of the block size %d", (long long)K, ti.vpb);
    if (N == 0) return GQ_OK;
    if (!dW || !dOut) return fail(GQ_ERR_INVALID, "gq_dequantize: null device pointer");
    if (!aligned_to(dW, 16) || !aligned_to(dOut, 16))
        return fail(GQ_ERR_INVALID, "gq_dequantize: weights and output must be 16-byte aligned");
    if (int rc = use_device()) return rc;
    return launch_dequantize(type, (const uint8_t *)dW, N, K, dOut, (hipStream_t)stream);
}

int gq_qdense_f32(int type, const float *dX, int64_t M, int64_t K, const void *dW, int64_t N, const float *dBias,
                  int act, float *dY, void *stream) {
    if (int rc = check_dense_args("gq_qdense_f32", type, dX, M, K, dW, N, dBias, act, dY, 4)) return rc;
    if (M == 0 || N == 0) return GQ_OK;
    if (int rc = use_device()) return rc;
    CallScope scope;
    // Small batches: GEMV passes cost about one third of the first pass per extra row; the split-K
    // MFMA kernels cost 19 .. 26 us (Q8_0 / Q4_0, K = 4096, N = 4096 .. 14336) for up to 32 rows and
    // 5 .. 18 us per further 32; the two passes 33 .. 62 us for anything up to 128 rows.  Measured
    // crossovers: split_k_from() / split_k_to().
    const bool tp = gemm_two_pass_supported(type, false, M, K, N, dX);
    const bool ks = M <= kGemvMaxRows && gemv_ks_supported(type, K, N, dX);
    const bool sk = M >= split_k_from(type, weight_bytes_of(type, K, N)) && mmq_supported(type, M, K, N, dX, dBias, dY) &&
                    (M <= split_k_to(type, K, N) || !tp);
    if (ks && !sk) return launch_gemv_ks(type, dX, false, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream);
    if (sk) return launch_mmq(type, dX, false, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream);
    // Shapes without a K-sliced plan (K not a multiple of 256: rare in models): a pass over W per row for up to 16
    // rows.  The 16-bit operands of the GEMMs below lean on averaging over many outputs and terms; on these few-row
    // problems seeded sweeps measured up to 0.9e-3 (1.25e-3 over a single block) through them, too close to the bound.
    if (M <= kGemvMaxRows) {
        if (gemv_xs_supported(type, K, N, dX))
            return launch_gemv_xs(type, dX, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream);
        return launch_gemv(type, dX, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream);
    }
    if (tp) return two_pass(type, false, dX, M, K, dW, N, dBias, act, dY, (hipStream_t)stream);
    return launch_gemm(type, false, dX, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream);
}

int gq_qdense_f32_static(int type, const float *dX, int64_t M, int64_t K, const void *dW, int64_t N, const float *dBias,
                         int act, float *dY, void *stream) {
    if (int rc = check_dense_args("gq_qdense_f32_static", type, dX, M, K, dW, N, dBias, act, dY, 4)) return rc;
    if (M == 0 || N == 0) return GQ_OK;
    if (int rc = use_device()) return rc;
    if (profile_state().active) return fail(GQ_ERR_INVALID, "gq_qdense_f32_static: kernel timing creates events; not available on this entry point");
    if (t_scope) return fail(GQ_ERR_INVALID, "gq_qdense_f32_static: not callable from inside another entry point");
    unsigned char *sp = static_cast<unsigned char *>(g_scratch_ptr[g_device.load(std::memory_order_acquire)]);
    if (!sp) return fail(GQ_ERR_NO_DEVICE, "gq_qdense_f32_static: gq_init() has not taken the scratch array's address on this device");
    CallScope scope;
    scope.static_ptr = sp;  // every scratch request below is served from the static array, or fails
    return gq_qdense_f32(type, dX, M, K, dW, N, dBias, act, dY, stream);
}

namespace {
bool takes_shared_pass(int count, const gq_dense_desc *descs, const float *gain, MmqSetItem *set);  // (defined with the dispatch thresholds below)
// From 6 rows the shared split-K pass is ahead of the merged GEMV launch: a decoder layer's q / k / v, 4096 -> 4096 + 2 x 1024,
// with the rest of the layer: 79.2 against 80.0 us at 5 rows, 81.6 against 79.9 at 6, 84.7 against 80.3 at 8.
constexpr int64_t kSharedPassFromRows = 6;
}  // namespace

int gq_qdense_f32_batch(int count, const gq_dense_desc *descs, void *stream) {
    if (count < 0 || (count > 0 && !descs)) return fail(GQ_ERR_INVALID, "gq_qdense_f32_batch: bad descriptor list");
    for (int i = 0; i < count; i++) {
        const gq_dense_desc &d = descs[i];
        if (int rc = check_dense_args("gq_qdense_f32_batch", d.type, d.dX, d.M, d.K, d.dW, d.N, d.dBias, d.act, d.dY, 4)) return rc;
    }
    if (count == 0) return GQ_OK;
    if (int rc = use_device()) return rc;
    CallScope scope;
    {   // projections of one input beyond the GEMV's best rows: one split-K pass for all of them
        MmqSetItem set[4];
        if (descs[0].M >= kSharedPassFromRows && takes_shared_pass(count, descs, nullptr, set))
            return launch_mmq_set(descs[0].type, descs[0].dX, false, descs[0].M, descs[0].K, count, set, nullptr, (hipStream_t)stream);
    }
    // merge runs of batch-1 problems of one type that the streaming GEMV handles; the rest go one by one
    int i = 0;
    while (i < count) {
        int j = i;
        XsBatchItem items[8];
        // the kernel family of the run is that of its first problem: K-sliced where that applies, else
        // activation-stationary
        const bool use_ks = gemv_ks_supported(descs[i].type, descs[i].K, descs[i].N, descs[i].dX);
        auto fits = [&](const gq_dense_desc &d) {
            return use_ks ? gemv_ks_supported(d.type, d.K, d.N, d.dX) : gemv_xs_supported(d.type, d.K, d.N, d.dX);
        };
        const int64_t rows = descs[i].M;
        const bool rows_ok = rows == 1 || (use_ks && rows >= 1 && rows <= batch_rows_max());
        // (several rows per problem: only over matrices below the size from which one pass serves several rows)
        auto size_ok = [&](const gq_dense_desc &d) { return rows == 1 || weight_bytes_of(d.type, d.K, d.N) < kLargeWeightBytes; };
        while (j < count && j - i < 8 && rows_ok && descs[j].type == descs[i].type && descs[j].M == rows && descs[j].N > 0 && fits(descs[j]) &&
               size_ok(descs[j])) {
            const gq_dense_desc &d = descs[j];
            items[j - i] = XsBatchItem{d.dX, (const uint8_t *)d.dW, d.dBias, d.dY, d.K, d.N, d.act};
            j++;
        }
        if (j - i >= 2) {
            if (int rc = use_ks ? launch_gemv_ks_batch(descs[i].type, j - i, items, (hipStream_t)stream, (int)rows)
                                : launch_gemv_xs_batch(descs[i].type, j - i, items, (hipStream_t)stream))
                return rc;
            i = j;
            continue;
        }
        const gq_dense_desc &d = descs[i];
        if (int rc = gq_qdense_f32(d.type, d.dX, d.M, d.K, d.dW, d.N, d.dBias, d.act, d.dY, stream)) return rc;
        i++;
    }
    return GQ_OK;
}

int gq_qdense_bf16(int type, const uint16_t *dX, int64_t M, int64_t K, const void *dW, int64_t N,
                   const float *dBias, int act, float *dY, void *stream) {
    if (int rc = check_dense_args("gq_qdense_bf16", type, dX, M, K, dW, N, dBias, act, dY, 2)) return rc;
    if (M == 0 || N == 0) return GQ_OK;
    if (int rc = use_device()) return rc;
    CallScope scope;
    // Same crossovers as for fp32 activations: bf16 widens exactly to fp32 for the GEMV passes and to
    // the fp16 activation image of the split-K kernels (which have no bf16 rounding of W: tighter than
    // the bf16 MFMA paths).
    const bool tp = gemm_two_pass_supported(type, true, M, K, N, dX);
    const bool ks = M <= kGemvMaxRows && gemv_ks_supported(type, K, N, dX);
    const bool sk = M >= split_k_from(type, weight_bytes_of(type, K, N)) && mmq_supported(type, M, K, N, dX, dBias, dY) &&
                    (M <= split_k_to(type, K, N) || !tp);
    if (ks && !sk) return launch_gemv_ks(type, dX, true, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream);
    if (sk) return launch_mmq(type, dX, true, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream);
    if (tp) return two_pass(type, true, dX, M, K, dW, N, dBias, act, dY, (hipStream_t)stream);
    return launch_gemm(type, true, dX, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream);
}

int gq_rmsnorm_f32(const float *dX, int64_t M, int64_t K, const float *dGain, float eps, float gain_offset, float *dY, void *stream) {
    if (M < 0 || K <= 0 || K > INT32_MAX) return fail(GQ_ERR_INVALID, "gq_rmsnorm_f32: bad shape [%lld, %lld]", (long long)M, (long long)K);
    if (!(eps >= 0.f)) return fail(GQ_ERR_INVALID, "gq_rmsnorm_f32: epsilon must be >= 0");
    if (M == 0) return GQ_OK;
    if (M > INT32_MAX) return fail(GQ_ERR_NOT_IMPLEMENTED, "gq_rmsnorm_f32: more than 2^31 - 1 rows");
    if (!dX || !dY) return fail(GQ_ERR_INVALID, "gq_rmsnorm_f32: null device pointer");
    if (!aligned_to(dX, 4) || !aligned_to(dY, 4) || (dGain && !aligned_to(dGain, 4)))
        return fail(GQ_ERR_INVALID, "gq_rmsnorm_f32: pointers must be 4-byte aligned");
    if (int rc = use_device()) return rc;
    return launch_rmsnorm(dX, M, K, dGain, gain_offset, eps, dY, (hipStream_t)stream);
}

namespace {
// First batch size at which a projection with its neighbours leaves the GEMV for the split-K kernels.  The GEMV with
// the extras walks a large matrix once per two rows (not four), the split-K form costs the same for any batch up to 32
// rows and carries the normalisation and the residual at no extra launch.  Measured (us per call in a replayed graph,
// RMSNorm in front; rows 2 3 4 5 6 7 8 on the GEMV | split-K):
//   block (one projection + residual)                                    gated pair (SiLU)
//   Q8_0   4096x4096 10 14 16 19 22 25 28 | 15   4096x14336 16 26 26 36 36 47 47 | 30      12 19 19 26 26 33 33 | 23   28 46 45 62 62 80 80 | 52
//   Q4_0   4096x4096  9 12 14 17 20 22 25 | 13   4096x14336 12 20 20 28 28 36 36 | 25      10 12 14 16 18 20 22 | 20   19 33 32 46 46 59 59 | 41
//   Q4_K   4096x4096  9 12 15 18 20 23 26 | 13   4096x14336 13 22 22 31 31 40 40 | 19      10 12 15 17 20 22 24 | 21   21 36 35 50 50 65 65 | 33
//   Q6_K   4096x4096 11 14 17 20 23 26 30 | 19   4096x14336 16 28 28 39 39 51 51 | 33      12 20 20 28 28 35 35 | 31   29 47 47 64 64 83 83 | 59
//   IQ4_NL 4096x4096 10 13 16 19 22 25 28 | 14   4096x14336 14 25 25 35 35 46 46 | 28      12 15 18 21 24 27 31 | 19   24 42 41 59 59 77 77 | 46
// (14336x4096 behaves like 4096x14336.)  Matrices of a few megabytes stay on the GEMV for every batch it takes.
int64_t block_split_k_from(int type, int64_t weight_bytes, bool gated) {
    if (weight_bytes < kTinyWeightBytes) return kGemvMaxRows + 1;
    if (weight_bytes >= kLargeWeightBytes) return type == GQ_Q4_K ? 3 : 5;
    switch (type) {
    case GQ_Q8_0: return gated ? 5 : 4;
    case GQ_Q4_0: return gated ? 8 : 5;
    case GQ_Q4_K: return gated ? 7 : 4;
    case GQ_Q6_K: return gated ? 7 : 5;
    case GQ_IQ4_NL: return gated ? 5 : 4;
    default: return 8;
    }
}

bool fold_into_gemv(int type, int64_t M, int64_t K, int64_t N, const float *x, const float *gain, const float *bias, const float *y, bool gated) {
    if (!gemv_ks_ext_supported(type, M, K, N, x, gain)) return false;
    return !(M >= block_split_k_from(type, weight_bytes_of(type, K, N), gated) && mmq_supported(type, M, K, N, x, bias, y));
}

// Whether a projection with its neighbours runs on the split-K kernels (after fold_into_gemv() has declined).
bool block_takes_split_k(int type, int64_t M, int64_t K, int64_t N, const float *x, const float *bias, const float *y, bool gated) {
    const bool tp = gated ? gemm_two_pass_block_supported(type, M, K, N, x, true) : gemm_two_pass_supported(type, false, M, K, N, x);
    const int64_t to = gated ? gated_split_k_to(type, K, N) : split_k_to(type, K, N);
    return M >= block_split_k_from(type, weight_bytes_of(type, K, N), gated) && mmq_supported(type, M, K, N, x, bias, y) && (M <= to || !tp);
}

// Whether a plain dense call on these operands runs on the split-K kernels (the dispatch of gq_qdense_f32).
bool dense_takes_split_k(int type, int64_t M, int64_t K, int64_t N, const float *x, const float *bias, const float *y) {
    const bool tp = gemm_two_pass_supported(type, false, M, K, N, x);
    return M >= split_k_from(type, weight_bytes_of(type, K, N)) && mmq_supported(type, M, K, N, x, bias, y) && (M <= split_k_to(type, K, N) || !tp);
}

// First batch size of the gated pair as one GEMM (wherever the split-K kernels have handed over: the composed form is never
// ahead); GOMLX_HIPQ_GATED_TWO_PASS_FROM=rows overrides it (tuning runs only).
int64_t gated_two_pass_from() {
    static const int64_t v = [] { const char *e = std::getenv("GOMLX_HIPQ_GATED_TWO_PASS_FROM"); return e ? (int64_t)std::atoll(e) : (int64_t)(kGemvMaxRows + 1); }();
    return v;
}

// Batches that a plain dense call would hand to the two-pass GEMM take its block form: the
// normalisation rides on the activation pass, the residual and the gated product on the epilogue.
bool block_takes_two_pass(int type, int64_t M, int64_t K, int64_t N, const float *x, const float *gain, const float *bias, const float *y,
                          bool gated) {
    if (M <= kGemvMaxRows || !gemm_two_pass_block_supported(type, M, K, N, x, gated)) return false;
    if (gated && M < gated_two_pass_from()) return false;
    if (gain && !aligned_to(gain, 16)) return false;
    const int64_t to = gated ? gated_split_k_to(type, K, N) : split_k_to(type, K, N);
    const bool sk = M >= split_k_from(type, weight_bytes_of(type, K, N)) && mmq_supported(type, M, K, N, x, bias, y) && M <= to;
    return !sk;
}
// Whether a list of projections is one input contracted with two to four matrices that the shared split-K pass takes
// (launch_mmq_set): equal type, activations, rows and K, the matrices taken together in the split-K kernels' range.
// Whether a list of two to four projections reads one input: equal type, activations, rows and K (fills `set`).
bool same_input_set(int count, const gq_dense_desc *descs, MmqSetItem *set) {
    if (count < 2 || count > 4) return false;
    for (int i = 0; i < count; i++) {
        const gq_dense_desc &d = descs[i];
        if (d.type != descs[0].type || d.dX != descs[0].dX || d.M != descs[0].M || d.K != descs[0].K || d.N <= 0) return false;
        set[i] = MmqSetItem{(const uint8_t *)d.dW, d.N, d.dBias, d.act, d.dY};
    }
    return true;
}
bool takes_shared_pass(int count, const gq_dense_desc *descs, const float *gain, MmqSetItem *set) {
    if ((gain && !aligned_to(gain, 16)) || !same_input_set(count, descs, set)) return false;
    const int type = descs[0].type;
    const int64_t rows = descs[0].M, K = descs[0].K;
    int64_t ntot = 0;
    for (int i = 0; i < count; i++) ntot += descs[i].N;
    return mmq_set_supported(type, count, set, rows, K, descs[0].dX) &&
           rows >= block_split_k_from(type, weight_bytes_of(type, K, ntot), false) &&
           (rows <= split_k_to(type, K, ntot) || !gemm_two_pass_supported(type, false, rows, K, ntot, descs[0].dX));
}
}  // namespace

int gq_qdense_block_f32(int type, const float *dX, int64_t M, int64_t K, const gq_rmsnorm *norm, const void *dW, int64_t N,
                        const float *dBias, int act, const float *dResidual, float *dY, void *stream) {
    if (!norm && !dResidual) return gq_qdense_f32(type, dX, M, K, dW, N, dBias, act, dY, stream);
    if (int rc = check_dense_args("gq_qdense_block_f32", type, dX, M, K, dW, N, dBias, act, dY, 4)) return rc;
    if (norm && !(norm->eps >= 0.f)) return fail(GQ_ERR_INVALID, "gq_qdense_block_f32: epsilon must be >= 0");
    if (norm && norm->dGain && !aligned_to(norm->dGain, 4)) return fail(GQ_ERR_INVALID, "gq_qdense_block_f32: gain must be 4-byte aligned");
    if (dResidual && !aligned_to(dResidual, 4)) return fail(GQ_ERR_INVALID, "gq_qdense_block_f32: residual must be 4-byte aligned");
    if (M == 0 || N == 0) return GQ_OK;
    if (int rc = use_device()) return rc;
    CallScope scope;
    RmsNorm rn{nullptr, 0.f, 0.f};
    if (norm) rn = RmsNorm{norm->dGain, norm->eps, norm->gain_offset};
    if (fold_into_gemv(type, M, K, N, dX, rn.gain, dBias, dY, false))
        return launch_gemv_ks_ext(type, dX, false, M, K, norm ? &rn : nullptr, (const uint8_t *)dW, dBias, nullptr, nullptr, dResidual, N, act, dY,
                                  (hipStream_t)stream);
    if (block_takes_two_pass(type, M, K, N, dX, rn.gain, dBias, dY, false)) {
        void *ws = nullptr;
        if (int rc = stream_workspace((hipStream_t)stream, gemm_two_pass_block_workspace(M, K, N, false), &ws)) return rc;
        return launch_gemm_two_pass_block(type, dX, M, K, norm ? &rn : nullptr, (const uint8_t *)dW, dBias, nullptr, nullptr, dResidual, N, act,
                                          dY, ws, (hipStream_t)stream);
    }
    // split-K range: the normalisation rides on the activation pre-pass and the reduction, the residual on the reduction
    if (block_takes_split_k(type, M, K, N, dX, dBias, dY, false) && (!dResidual || aligned_to(dResidual, 16)) && (!rn.gain || aligned_to(rn.gain, 16))) {
        const MmqExtra ex{nullptr, nullptr, dResidual, norm ? &rn : nullptr};
        return launch_mmq(type, dX, false, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream, &ex);
    }
    // composed: normalised activations into the stream's second workspace, the dense call, then the residual.  When y
    // overlaps the residual (a residual stream updated in place) the dense result goes to the workspace first: written
    // straight to y it would destroy the residual before the addition reads it.
    const float *x = dX;
    const size_t y_bytes = (size_t)M * (size_t)N * sizeof(float);
    const bool in_place = dResidual && reinterpret_cast<uintptr_t>(dY) < reinterpret_cast<uintptr_t>(dResidual) + y_bytes &&
                          reinterpret_cast<uintptr_t>(dResidual) < reinterpret_cast<uintptr_t>(dY) + y_bytes;
    const size_t xn_bytes = norm ? ((size_t)M * (size_t)K * sizeof(float) + 255) / 256 * 256 : 0;
    float *tmp = nullptr;
    if (norm || in_place) {
        void *ws = nullptr;
        if (int rc = stream_workspace((hipStream_t)stream, xn_bytes + (in_place ? y_bytes : 0), &ws, 1)) return rc;
        tmp = reinterpret_cast<float *>(static_cast<uint8_t *>(ws) + xn_bytes);
        if (norm) {
            float *xn = static_cast<float *>(ws);
            if (int rc = launch_rmsnorm(dX, M, K, rn.gain, rn.gain_offset, rn.eps, xn, (hipStream_t)stream)) return rc;
            x = xn;
        }
    }
    if (dResidual && dense_takes_split_k(type, M, K, N, x, dBias, dY) && aligned_to(dResidual, 16)) {  // the residual rides on the reduction
        const MmqExtra ex{nullptr, nullptr, dResidual, nullptr};
        return launch_mmq(type, x, false, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream, &ex);
    }
    float *dense_out = in_place ? tmp : dY;
    if (int rc = gq_qdense_f32(type, x, M, K, dW, N, dBias, act, dense_out, stream)) return rc;
    if (dResidual) return launch_add(dense_out, dResidual, dY, M * N, (hipStream_t)stream);
    return GQ_OK;
}

namespace {
// Whether a list of projections behind one normalisation is one launch of the K-sliced GEMV: every problem a projection of one
// type, one K and one (small) batch size that kernel takes (dX may point at fp32 or bf16 data: only its alignment matters),
// unless the shared split-K pass takes them at that batch size.  Fills items[0 .. count).
bool merges_into_gemv(int count, const gq_dense_desc *descs, const gq_rmsnorm *norm, bool shared_pass, XsBatchItem *items) {
    const int64_t rows = descs[0].M;
    bool merged = count >= 2 && count <= 8 && rows >= 1 && rows <= batch_rows_max() && !(shared_pass && rows >= kSharedPassFromRows);
    for (int i = 0; i < count && merged; i++) {
        const gq_dense_desc &d = descs[i];
        merged = d.type == descs[0].type && d.K == descs[0].K && d.M == rows && d.N > 0 && gemv_ks_ext_supported(d.type, rows, d.K, d.N, d.dX, norm->dGain) &&
                 (rows == 1 || weight_bytes_of(d.type, d.K, d.N) < kLargeWeightBytes);
        if (merged) items[i] = XsBatchItem{d.dX, (const uint8_t *)d.dW, d.dBias, d.dY, d.K, d.N, d.act};
    }
    return merged;
}
}  // namespace

int gq_qdense_norm_f32_batch(int count, const gq_dense_desc *descs, const gq_rmsnorm *norm, void *stream) {
    if (!norm) return gq_qdense_f32_batch(count, descs, stream);
    if (count < 0 || (count > 0 && !descs)) return fail(GQ_ERR_INVALID, "gq_qdense_norm_f32_batch: bad descriptor list");
    for (int i = 0; i < count; i++) {
        const gq_dense_desc &d = descs[i];
        if (int rc = check_dense_args("gq_qdense_norm_f32_batch", d.type, d.dX, d.M, d.K, d.dW, d.N, d.dBias, d.act, d.dY, 4)) return rc;
    }
    if (!(norm->eps >= 0.f)) return fail(GQ_ERR_INVALID, "gq_qdense_norm_f32_batch: epsilon must be >= 0");
    if (count == 0) return GQ_OK;
    if (int rc = use_device()) return rc;
    CallScope scope;
    const int64_t rows = descs[0].M;
    // Projections of the same activations (q / k / v) can share one split-K pass - one activation image, one main launch
    // over all their rows, one reduction - where the matrices taken together are in that kernel's range (three calls
    // would convert the activations three times and pay nine launches).
    MmqSetItem set[4];
    const bool shared_pass = takes_shared_pass(count, descs, norm->dGain, set);
    XsBatchItem items[8];
    if (merges_into_gemv(count, descs, norm, shared_pass, items)) {
        const RmsNorm rn{norm->dGain, norm->eps, norm->gain_offset};
        return launch_gemv_ks_batch_norm(descs[0].type, count, items, &rn, (hipStream_t)stream, (int)rows);
    }
    if (shared_pass) {
        const RmsNorm rn{norm->dGain, norm->eps, norm->gain_offset};
        return launch_mmq_set(descs[0].type, descs[0].dX, false, rows, descs[0].K, count, set, &rn, (hipStream_t)stream);
    }
    // Past the split-K range the same projections share the two passes: one activation conversion, one image of all the
    // matrices, one GEMM (a decoder layer's q / k / v at 128 rows: two launches instead of six).
    if (same_input_set(count, descs, set) && rows > kGemvMaxRows && (!norm->dGain || aligned_to(norm->dGain, 16)) &&
        gemm_two_pass_set_supported(descs[0].type, count, set, rows, descs[0].K, descs[0].dX)) {
        void *ws = nullptr;
        if (int rc = stream_workspace((hipStream_t)stream, gemm_two_pass_set_workspace(count, set, rows, descs[0].K), &ws)) return rc;
        const RmsNorm rn{norm->dGain, norm->eps, norm->gain_offset};
        return launch_gemm_two_pass_set(descs[0].type, descs[0].dX, rows, descs[0].K, &rn, count, set, ws, (hipStream_t)stream);
    }
    for (int i = 0; i < count; i++) {
        const gq_dense_desc &d = descs[i];
        if (int rc = gq_qdense_block_f32(d.type, d.dX, d.M, d.K, norm, d.dW, d.N, d.dBias, d.act, nullptr, d.dY, stream)) return rc;
    }
    return GQ_OK;
}

int gq_qdense_gated_f32(int type, const float *dX, int64_t M, int64_t K, const gq_rmsnorm *norm, const void *dWgate,
                        const float *dBiasGate, const void *dWup, const float *dBiasUp, int64_t N, int act, float *dY, void *stream) {
    if (int rc = check_dense_args("gq_qdense_gated_f32", type, dX, M, K, dWgate, N, dBiasGate, act, dY, 4)) return rc;
    if (int rc = check_dense_args("gq_qdense_gated_f32", type, dX, M, K, dWup, N, dBiasUp, act, dY, 4)) return rc;
    if (norm && !(norm->eps >= 0.f)) return fail(GQ_ERR_INVALID, "gq_qdense_gated_f32: epsilon must be >= 0");
    if (norm && norm->dGain && !aligned_to(norm->dGain, 4)) return fail(GQ_ERR_INVALID, "gq_qdense_gated_f32: gain must be 4-byte aligned");
    if (M == 0 || N == 0) return GQ_OK;
    if (int rc = use_device()) return rc;
    CallScope scope;
    RmsNorm rn{nullptr, 0.f, 0.f};
    if (norm) rn = RmsNorm{norm->dGain, norm->eps, norm->gain_offset};
    if (fold_into_gemv(type, M, K, N, dX, rn.gain, dBiasGate, dY, true))
        return launch_gemv_ks_ext(type, dX, false, M, K, norm ? &rn : nullptr, (const uint8_t *)dWgate, dBiasGate, (const uint8_t *)dWup, dBiasUp,
                                  nullptr, N, act, dY, (hipStream_t)stream);
    if (block_takes_two_pass(type, M, K, N, dX, rn.gain, dBiasGate, dY, true)) {
        void *ws = nullptr;
        if (int rc = stream_workspace((hipStream_t)stream, gemm_two_pass_block_workspace(M, K, N, true), &ws)) return rc;
        return launch_gemm_two_pass_block(type, dX, M, K, norm ? &rn : nullptr, (const uint8_t *)dWgate, dBiasGate, (const uint8_t *)dWup, dBiasUp,
                                          nullptr, N, act, dY, ws, (hipStream_t)stream);
    }
    if (block_takes_split_k(type, M, K, N, dX, dBiasGate, dY, true) && (!dBiasUp || aligned_to(dBiasUp, 16)) && (!rn.gain || aligned_to(rn.gain, 16))) {
        // both matrices against one activation image (which carries the gain); the reduction normalises and forms act(gate) * up
        const MmqExtra ex{(const uint8_t *)dWup, dBiasUp, nullptr, norm ? &rn : nullptr};
        return launch_mmq(type, dX, false, M, K, (const uint8_t *)dWgate, N, dBiasGate, act, dY, (hipStream_t)stream, &ex);
    }
    // composed: [normalised activations,] act(gate) into the stream's second workspace, up into y, y *= act(gate)
    const size_t xn_bytes = norm ? ((size_t)M * (size_t)K * sizeof(float) + 255) / 256 * 256 : 0;
    void *ws = nullptr;
    if (int rc = stream_workspace((hipStream_t)stream, xn_bytes + (size_t)M * (size_t)N * sizeof(float), &ws, 1)) return rc;
    const float *x = dX;
    if (norm) {
        float *xn = static_cast<float *>(ws);
        if (int rc = launch_rmsnorm(dX, M, K, rn.gain, rn.gain_offset, rn.eps, xn, (hipStream_t)stream)) return rc;
        x = xn;
    }
    if (dense_takes_split_k(type, M, K, N, x, dBiasGate, dY) && (!dBiasUp || aligned_to(dBiasUp, 16))) {
        // both matrices against one activation image; the reduction forms act(gate) * up
        const MmqExtra ex{(const uint8_t *)dWup, dBiasUp, nullptr, nullptr};
        return launch_mmq(type, x, false, M, K, (const uint8_t *)dWgate, N, dBiasGate, act, dY, (hipStream_t)stream, &ex);
    }
    float *gate = reinterpret_cast<float *>(static_cast<uint8_t *>(ws) + xn_bytes);
    if (int rc = gq_qdense_f32(type, x, M, K, dWgate, N, dBiasGate, act, gate, stream)) return rc;
    if (int rc = gq_qdense_f32(type, x, M, K, dWup, N, dBiasUp, GQ_ACT_NONE, dY, stream)) return rc;
    return launch_mul_inplace(dY, gate, M * N, (hipStream_t)stream);
}

// ---- the same callers with bf16 activations: the decode GEMV reads them as they are (widened in registers: exact); the other
// routes get them widened to fp32 in the stream's third workspace ----
namespace {
// fp32 copy of a bf16 [M, K] matrix at `offset` bytes into the widening workspace, whose size the caller has fixed
int widen_into(void *ws, size_t offset, const uint16_t *x, int64_t M, int64_t K, hipStream_t s, const float **out) {
    float *dst = reinterpret_cast<float *>(static_cast<uint8_t *>(ws) + offset);
    if (int rc = launch_widen_bf16(x, dst, M * K, s)) return rc;
    *out = dst;
    return GQ_OK;
}
size_t widened_bytes(int64_t M, int64_t K) { return ((size_t)M * (size_t)K * sizeof(float) + 255) & ~(size_t)255; }
}  // namespace

int gq_qdense_block_bf16(int type, const uint16_t *dX, int64_t M, int64_t K, const gq_rmsnorm *norm, const void *dW, int64_t N,
                         const float *dBias, int act, const float *dResidual, float *dY, void *stream) {
    if (!norm && !dResidual) return gq_qdense_bf16(type, dX, M, K, dW, N, dBias, act, dY, stream);
    if (int rc = check_dense_args("gq_qdense_block_bf16", type, dX, M, K, dW, N, dBias, act, dY, 16)) return rc;
    if (norm && !(norm->eps >= 0.f)) return fail(GQ_ERR_INVALID, "gq_qdense_block_bf16: epsilon must be >= 0");
    if (norm && norm->dGain && !aligned_to(norm->dGain, 4)) return fail(GQ_ERR_INVALID, "gq_qdense_block_bf16: gain must be 4-byte aligned");
    if (dResidual && !aligned_to(dResidual, 4)) return fail(GQ_ERR_INVALID, "gq_qdense_block_bf16: residual must be 4-byte aligned");
    if (M == 0 || N == 0) return GQ_OK;
    if (int rc = use_device()) return rc;
    CallScope scope;
    if (fold_into_gemv(type, M, K, N, reinterpret_cast<const float *>(dX), norm ? norm->dGain : nullptr, dBias, dY, false)) {
        const RmsNorm rn = norm ? RmsNorm{norm->dGain, norm->eps, norm->gain_offset} : RmsNorm{nullptr, 0.f, 0.f};
        return launch_gemv_ks_ext(type, dX, true, M, K, norm ? &rn : nullptr, (const uint8_t *)dW, dBias, nullptr, nullptr, dResidual, N, act, dY,
                                  (hipStream_t)stream);
    }
    {   // the split-K kernels' pre-pass reads bf16 as well (where the fp32 call would take them too)
        const float *xa = reinterpret_cast<const float *>(dX), *gain = norm ? norm->dGain : nullptr;  // (only their alignment is looked at)
        if (!block_takes_two_pass(type, M, K, N, xa, gain, dBias, dY, false) && block_takes_split_k(type, M, K, N, xa, dBias, dY, false) &&
            (!dResidual || aligned_to(dResidual, 16)) && (!gain || aligned_to(gain, 16))) {
            const RmsNorm rn = norm ? RmsNorm{norm->dGain, norm->eps, norm->gain_offset} : RmsNorm{nullptr, 0.f, 0.f};
            const MmqExtra ex{nullptr, nullptr, dResidual, norm ? &rn : nullptr};
            return launch_mmq(type, dX, true, M, K, (const uint8_t *)dW, N, dBias, act, dY, (hipStream_t)stream, &ex);
        }
    }
    void *ws = nullptr;
    if (int rc = stream_workspace((hipStream_t)stream, widened_bytes(M, K), &ws, kWsWidenSlot)) return rc;
    const float *x32 = nullptr;
    if (int rc = widen_into(ws, 0, dX, M, K, (hipStream_t)stream, &x32)) return rc;
    return gq_qdense_block_f32(type, x32, M, K, norm, dW, N, dBias, act, dResidual, dY, stream);
}

int gq_qdense_gated_bf16(int type, const uint16_t *dX, int64_t M, int64_t K, const gq_rmsnorm *norm, const void *dWgate,
                         const float *dBiasGate, const void *dWup, const float *dBiasUp, int64_t N, int act, float *dY, void *stream) {
    if (int rc = check_dense_args("gq_qdense_gated_bf16", type, dX, M, K, dWgate, N, dBiasGate, act, dY, 16)) return rc;
    if (int rc = check_dense_args("gq_qdense_gated_bf16", type, dX, M, K, dWup, N, dBiasUp, act, dY, 16)) return rc;
    if (norm && !(norm->eps >= 0.f)) return fail(GQ_ERR_INVALID, "gq_qdense_gated_bf16: epsilon must be >= 0");
    if (norm && norm->dGain && !aligned_to(norm->dGain, 4)) return fail(GQ_ERR_INVALID, "gq_qdense_gated_bf16: gain must be 4-byte aligned");
    if (M == 0 || N == 0) return GQ_OK;
    if (int rc = use_device()) return rc;
    CallScope scope;
    if (fold_into_gemv(type, M, K, N, reinterpret_cast<const float *>(dX), norm ? norm->dGain : nullptr, dBiasGate, dY, true)) {
        const RmsNorm rn = norm ? RmsNorm{norm->dGain, norm->eps, norm->gain_offset} : RmsNorm{nullptr, 0.f, 0.f};
        return launch_gemv_ks_ext(type, dX, true, M, K, norm ? &rn : nullptr, (const uint8_t *)dWgate, dBiasGate, (const uint8_t *)dWup, dBiasUp, nullptr,
                                  N, act, dY, (hipStream_t)stream);
    }
    {
        const float *xa = reinterpret_cast<const float *>(dX), *gain = norm ? norm->dGain : nullptr;  // (only their alignment is looked at)
        if (!block_takes_two_pass(type, M, K, N, xa, gain, dBiasGate, dY, true) && block_takes_split_k(type, M, K, N, xa, dBiasGate, dY, true) &&
            (!dBiasUp || aligned_to(dBiasUp, 16)) && (!gain || aligned_to(gain, 16))) {
            const RmsNorm rn = norm ? RmsNorm{norm->dGain, norm->eps, norm->gain_offset} : RmsNorm{nullptr, 0.f, 0.f};
            const MmqExtra ex{(const uint8_t *)dWup, dBiasUp, nullptr, norm ? &rn : nullptr};
            return launch_mmq(type, dX, true, M, K, (const uint8_t *)dWgate, N, dBiasGate, act, dY, (hipStream_t)stream, &ex);
        }
    }
    void *ws = nullptr;
    if (int rc = stream_workspace((hipStream_t)stream, widened_bytes(M, K), &ws, kWsWidenSlot)) return rc;
    const float *x32 = nullptr;
    if (int rc = widen_into(ws, 0, dX, M, K, (hipStream_t)stream, &x32)) return rc;
    return gq_qdense_gated_f32(type, x32, M, K, norm, dWgate, dBiasGate, dWup, dBiasUp, N, act, dY, stream);
}

int gq_qdense_norm_bf16_batch(int count, const gq_dense_desc *descs, const gq_rmsnorm *norm, void *stream) {
    if (count < 0 || (count > 0 && !descs)) return fail(GQ_ERR_INVALID, "gq_qdense_norm_bf16_batch: bad descriptor list");
    if (count > 64) return fail(GQ_ERR_NOT_IMPLEMENTED, "gq_qdense_norm_bf16_batch: more than 64 problems in one submission");
    for (int i = 0; i < count; i++) {
        const gq_dense_desc &d = descs[i];
        if (int rc = check_dense_args("gq_qdense_norm_bf16_batch", d.type, d.dX, d.M, d.K, d.dW, d.N, d.dBias, d.act, d.dY, 16)) return rc;
    }
    if (norm && !(norm->eps >= 0.f)) return fail(GQ_ERR_INVALID, "gq_qdense_norm_bf16_batch: epsilon must be >= 0");
    if (count == 0) return GQ_OK;
    if (int rc = use_device()) return rc;
    CallScope scope;
    if (norm && count <= 8) {  // the list as one launch of the decode GEMV, on the bf16 data as it is
        MmqSetItem set[4];
        const bool shared_pass = takes_shared_pass(count, descs, norm->dGain, set);
        XsBatchItem items[8];
        if (merges_into_gemv(count, descs, norm, shared_pass, items)) {
            const RmsNorm rn{norm->dGain, norm->eps, norm->gain_offset};
            return launch_gemv_ks_batch_norm(descs[0].type, count, items, &rn, (hipStream_t)stream, (int)descs[0].M, true);
        }
        if (shared_pass) {
            const RmsNorm rn{norm->dGain, norm->eps, norm->gain_offset};
            return launch_mmq_set(descs[0].type, descs[0].dX, true, descs[0].M, descs[0].K, count, set, &rn, (hipStream_t)stream);
        }
    }
    // every distinct activation matrix (q / k / v share theirs) is widened once
    gq_dense_desc wide[64];
    size_t offset[64], total = 0;
    int first[64];
    for (int i = 0; i < count; i++) {
        first[i] = -1;  // an empty problem (no rows or no columns) reads no activations: it neither gets nor lends a widened copy
        if (descs[i].M == 0 || descs[i].N == 0) continue;
        first[i] = i;
        for (int j = 0; j < i; j++)
            if (first[j] >= 0 && descs[j].dX == descs[i].dX && descs[j].M == descs[i].M && descs[j].K == descs[i].K) { first[i] = first[j]; break; }
        if (first[i] == i) { offset[i] = total; total += widened_bytes(descs[i].M, descs[i].K); }
    }
    void *ws = nullptr;
    if (total)
        if (int rc = stream_workspace((hipStream_t)stream, total, &ws, kWsWidenSlot)) return rc;
    for (int i = 0; i < count; i++) {
        wide[i] = descs[i];
        if (first[i] < 0) continue;
        if (first[i] == i) {
            const float *x32 = nullptr;
            if (int rc = widen_into(ws, offset[i], reinterpret_cast<const uint16_t *>(descs[i].dX), descs[i].M, descs[i].K, (hipStream_t)stream, &x32)) return rc;
            wide[i].dX = x32;
        } else {
            wide[i].dX = wide[first[i]].dX;
        }
    }
    return gq_qdense_norm_f32_batch(count, wide, norm, stream);
}

int gq_embedding_lookup(int type, const void *dTable, int64_t vocab, int64_t K, const int32_t *dIndices,
                        int64_t count, float *dOut, int32_t *dErrFlag, void *stream) {
    TypeInfo ti;
    if (!type_info(type, ti)) return fail(GQ_ERR_NOT_IMPLEMENTED, "gq_embedding_lookup: ggml type %d is not implemented", type);
    if (vocab < 0 || count < 0) return fail(GQ_ERR_INVALID, "gq_embedding_lookup: negative size");
    if (K <= 0 || K % ti.vpb != 0)
        return fail(GQ_ERR_INVALID, "gq_embedding_lookup: K=%lld is not a positive multiple of the block size %d", (long long)K, ti.vpb);
    if (count == 0) return GQ_OK;
    if (vocab == 0) return fail(GQ_ERR_INVALID, "gq_embedding_lookup: empty table with %lld indices", (long long)count);
    if (!dTable || !dIndices || !dOut) return fail(GQ_ERR_INVALID, "gq_embedding_lookup: null device pointer");
    if (!aligned_to(dTable, 16) || !aligned_to(dOut, 16) || !aligned_to(dIndices, 4))
        return fail(GQ_ERR_INVALID, "gq_embedding_lookup: table and output must be 16-byte aligned");
    if (int rc = use_device()) return rc;
    return launch_embedding_lookup(type, (const uint8_t *)dTable, vocab, K, dIndices, count, dOut, dErrFlag,
                                   (hipStream_t)stream);
}

int gq_graph_begin(void *stream) {
    if (!stream) return fail(GQ_ERR_INVALID, "gq_graph_begin: recording needs an explicit stream");
    if (profile_state().active) return fail(GQ_ERR_INVALID, "gq_graph_begin: kernel timing is active on this thread");
    if (int rc = use_device()) return rc;
    pool().begin_recording(stream);
    GQ_HIP(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return GQ_OK;
}

int gq_graph_end(void *stream, void **graph_exec) {
    if (!stream || !graph_exec) return fail(GQ_ERR_INVALID, "gq_graph_end: null argument");
    *graph_exec = nullptr;
    if (int rc = use_device()) return rc;
    hipGraph_t graph = nullptr;
    const hipError_t ce = hipStreamEndCapture((hipStream_t)stream, &graph);
    std::vector<WsBlockRef> blocks = pool().end_recording(stream);  // the workspaces the recorded launches point at
    if (ce != hipSuccess) { pool().unpin(blocks); return hip_fail(ce, "hipStreamEndCapture"); }
    hipGraphExec_t exec = nullptr;
    const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) { pool().unpin(blocks); return hip_fail(e, "hipGraphInstantiate"); }
    RecordedGraph *g = new (std::nothrow) RecordedGraph;
    if (!g) { (void)hipGraphExecDestroy(exec); pool().unpin(blocks); return fail(GQ_ERR_OOM, "gq_graph_end: out of host memory"); }
    g->exec = exec;
    g->stream = (hipStream_t)stream;
    g->blocks.swap(blocks);
    *graph_exec = g;
    return GQ_OK;
}

int gq_graph_launch(void *graph_exec, void *stream) {
    if (!graph_exec) return fail(GQ_ERR_INVALID, "gq_graph_launch: null graph");
    RecordedGraph *g = static_cast<RecordedGraph *>(graph_exec);
    // The recorded launches point at the recording stream's workspace, which eager calls on that stream share in
    // stream order: a replay on another stream would run unordered against them.
    if ((hipStream_t)stream != g->stream)
        return fail(GQ_ERR_INVALID, "gq_graph_launch: a graph replays on the stream it was recorded on");
    if (int rc = use_device()) return rc;
    // (replays and eager sequences that share the workspace must not interleave their submissions)
    WsStreamRef st = pool().stream(stream);
    std::lock_guard<std::recursive_mutex> seq(st->seq);
    GQ_HIP(hipGraphLaunch(g->exec, g->stream));
    return GQ_OK;
}

int gq_graph_destroy(void *graph_exec) {
    if (!graph_exec) return GQ_OK;
    if (int rc = use_device()) return rc;
    RecordedGraph *g = static_cast<RecordedGraph *>(graph_exec);
    const hipError_t e = hipGraphExecDestroy(g->exec);
    pool().unpin(g->blocks);
    delete g;
    if (e != hipSuccess) return hip_fail(e, "hipGraphExecDestroy");
    return GQ_OK;
}

int gq_profile_begin(void) {
    ProfileState &ps = profile_state();
    if (ps.active) return fail(GQ_ERR_INVALID, "gq_profile_begin: already active on this thread");
    if (int rc = use_device()) return rc;
    ps.active = true;
    ps.events.clear();
    return GQ_OK;
}

int gq_profile_end(int *launches, double *total_us) {
    ProfileState &ps = profile_state();
    if (!ps.active) return fail(GQ_ERR_INVALID, "gq_profile_end: timing is not active on this thread");
    ps.active = false;
    int rc = use_device();
    double total = 0.0;
    int n = 0;
    for (size_t i = 0; i + 1 < ps.events.size(); i += 2) {
        if (rc == GQ_OK) {
            float ms = 0.f;
            hipError_t e = hipEventSynchronize(ps.events[i + 1]);
            if (e == hipSuccess) e = hipEventElapsedTime(&ms, ps.events[i], ps.events[i + 1]);
            if (e != hipSuccess) rc = hip_fail(e, "hipEventElapsedTime");
            else { total += (double)ms * 1000.0; n++; }
        }
        (void)hipEventDestroy(ps.events[i]);
        (void)hipEventDestroy(ps.events[i + 1]);
    }
    ps.events.clear();
    if (launches) *launches = n;
    if (total_us) *total_us = total;
    return rc;
}

int gq_workspace_stats(size_t *live_bytes, int *streams) {
    if (live_bytes) *live_bytes = pool().live_bytes();
    if (streams) *streams = (int)pool().stream_count();
    return GQ_OK;
}

const char *gq_last_error(void) { return g_error; }

}  // extern "C"
