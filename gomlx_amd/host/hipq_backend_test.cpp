// Tests of the C++ host layer, written the way the reference's Go tests of this path are:
// each case builds a graph with the nn.* operator, compiles it, executes it twice (the way
// graphtest.RunTestGraphFn does, core/graph/graphtest/graphtest.go:54-107) and compares the
// outputs with an absolute tolerance.  Cases and expected values follow
//   ml/nn/quantized_dense_test.go:272-452   (TestQuantizedDense_GGML_Q8_0 / _Q4_0 / _IQ4NL)
//   ml/nn/quantized_gather_test.go:17-169   (TestQuantizedGather_*)
//   core/graph/fused_ops.go:339-373         (the fallback rules of InternalFusedOpCaller; the reference holds no test of
//                                            its own for them, the cases here follow the function's documented contract)
//
// usage: hipq_backend_test [--build-only]
//   --build-only runs the cases that need no GPU (graph-build validation and fallback logic).
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "hipq_backend.hpp"

using namespace gomlx_hipq;

static int g_failed = 0, g_run = 0;
static std::string g_case;

#define CHECK(cond, ...)                                                            \
    do {                                                                            \
        if (!(cond)) {                                                              \
            std::printf("  FAIL %s (%s:%d): ", g_case.c_str(), __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                                               \
            std::printf("\n");                                                      \
            g_failed++;                                                             \
            return;                                                                 \
        }                                                                           \
    } while (0)

struct Tensor {
    Shape shape;
    std::vector<uint8_t> bytes;
    static Tensor F32(std::vector<int64_t> dims, const std::vector<float> &v) {
        Tensor t; t.shape = Shape{DType::Float32, std::move(dims)}; t.bytes.resize(v.size() * 4);
        std::memcpy(t.bytes.data(), v.data(), t.bytes.size()); return t;
    }
    static Tensor U8(std::vector<int64_t> dims, const std::vector<uint8_t> &v) {
        Tensor t; t.shape = Shape{DType::Uint8, std::move(dims)}; t.bytes = v; return t;
    }
    static Tensor I32(std::vector<int64_t> dims, const std::vector<int32_t> &v) {
        Tensor t; t.shape = Shape{DType::Int32, std::move(dims)}; t.bytes.resize(v.size() * 4);
        std::memcpy(t.bytes.data(), v.data(), t.bytes.size()); return t;
    }
};

using GraphFn = std::function<std::pair<std::vector<Value>, Error>(Function *, const std::vector<Value> &)>;

// Builds, compiles and runs `fn` over `inputs` twice; the outputs of both runs must match `want`.
static void RunTestGraphFn(Backend *backend, const std::string &name, const std::vector<Tensor> &inputs, const GraphFn &fn,
                           const std::vector<std::vector<float>> &want, double delta) {
    g_case = name; g_run++;
    auto builder = backend->Builder(name);
    std::vector<Value> params;
    for (size_t i = 0; i < inputs.size(); i++) {
        auto p = builder->Main()->Parameter("p" + std::to_string(i), inputs[i].shape);
        CHECK(p.second.ok(), "Parameter: %s", p.second.message.c_str());
        params.push_back(p.first);
    }
    auto outs = fn(builder->Main(), params);
    CHECK(outs.second.ok(), "graph function: %s", outs.second.message.c_str());
    Error e = builder->Main()->Return(outs.first);
    CHECK(e.ok(), "Return: %s", e.message.c_str());
    auto exec = builder->Compile();
    CHECK(exec.second.ok(), "Compile: %s", exec.second.message.c_str());
    std::vector<BufferPtr> bufs;
    for (const Tensor &t : inputs) {
        auto b = backend->BufferFromFlatData(0, t.bytes.data(), t.shape);
        CHECK(b.second.ok(), "BufferFromFlatData: %s", b.second.message.c_str());
        bufs.push_back(b.first);
    }
    for (int run = 0; run < 2; run++) {
        auto res = exec.first->Execute(bufs);
        CHECK(res.second.ok(), "Execute: %s", res.second.message.c_str());
        CHECK(res.first.size() == want.size(), "got %zu outputs, want %zu", res.first.size(), want.size());
        for (size_t o = 0; o < want.size(); o++) {
            std::vector<float> got((size_t)res.first[o]->GetShape().Size());
            CHECK(got.size() == want[o].size(), "output %zu has %zu elements, want %zu", o, got.size(), want[o].size());
            Error te = res.first[o]->ToFlatData(got.data());
            CHECK(te.ok(), "ToFlatData: %s", te.message.c_str());
            for (size_t i = 0; i < got.size(); i++)
                CHECK(std::fabs((double)got[i] - (double)want[o][i]) <= delta, "run %d output %zu [%zu]: got %g want %g (delta %g)", run, o, i,
                      got[i], want[o][i], delta);
        }
    }
    std::printf("  ok   %s\n", name.c_str());
}

// ---- block builders used by the reference tests -----------------------------------------------
static std::vector<uint8_t> Q8Row(uint8_t scaleHi, std::initializer_list<int> ones) {
    std::vector<uint8_t> r(34, 0); r[1] = scaleHi;
    for (int i : ones) r[2 + i] = 1;
    return r;
}
static std::vector<uint8_t> Q4Row(uint8_t scaleHi, int byteWith9) {
    std::vector<uint8_t> r(18, 0x88); r[0] = 0; r[1] = scaleHi; r[2 + byteWith9] = 0x89;
    return r;
}
static std::vector<uint8_t> Cat(std::initializer_list<std::vector<uint8_t>> rows) {
    std::vector<uint8_t> v;
    for (const auto &r : rows) v.insert(v.end(), r.begin(), r.end());
    return v;
}
static std::vector<float> Unit(std::initializer_list<std::pair<int, float>> nz, int n = 32) {
    std::vector<float> v((size_t)n, 0.f);
    for (auto p : nz) v[(size_t)p.first] = p.second;
    return v;
}
static Quantization GGML(GGMLQuantType t) { Quantization q; q.scheme = QuantScheme::GGML; q.ggmlType = t; return q; }

static GraphFn DenseFn(GGMLQuantType t, bool withBias, std::vector<activation::Type> act = {}) {
    return [=](Function *f, const std::vector<Value> &in) {
        Quantization q = GGML(t);
        auto r = nn::QuantizedDense(f, in[0], in[1], &q, withBias ? in[2] : Value(), act);
        return std::make_pair(std::vector<Value>{r.first}, r.second);
    };
}

static void TestQuantizedDenseGGML(Backend *b) {
    const std::vector<float> xBasic = Unit({{0, 1.f}, {1, 1.f}});
    std::vector<float> xBatch = xBasic;
    { auto h = Unit({{0, 0.5f}}); xBatch.insert(xBatch.end(), h.begin(), h.end()); }
    const auto q8w = Tensor::U8({2, 34}, Cat({Q8Row(0x40, {0}), Q8Row(0x42, {1})}));
    const auto q4w = Tensor::U8({2, 18}, Cat({Q4Row(0x40, 0), Q4Row(0x42, 1)}));
    const auto iqw = Tensor::U8({2, 18}, Cat({Q4Row(0x3C, 0), Q4Row(0x40, 1)}));
    RunTestGraphFn(b, "QuantizedDense_GGML_Q8_0/basic", {Tensor::F32({1, 32}, xBasic), q8w}, DenseFn(GGMLQuantType::Q8_0, false), {{2.f, 3.f}}, 1e-4);
    RunTestGraphFn(b, "QuantizedDense_GGML_Q8_0/with_bias", {Tensor::F32({1, 32}, xBasic), q8w, Tensor::F32({2}, {0.5f, -0.5f})},
                   DenseFn(GGMLQuantType::Q8_0, true), {{2.5f, 2.5f}}, 1e-4);
    RunTestGraphFn(b, "QuantizedDense_GGML_Q8_0/batch", {Tensor::F32({2, 32}, xBatch), q8w}, DenseFn(GGMLQuantType::Q8_0, false),
                   {{2.f, 3.f, 1.f, 0.f}}, 1e-4);
    RunTestGraphFn(b, "QuantizedDense_GGML_Q4_0/basic", {Tensor::F32({1, 32}, xBasic), q4w}, DenseFn(GGMLQuantType::Q4_0, false), {{2.f, 3.f}}, 1e-4);
    RunTestGraphFn(b, "QuantizedDense_GGML_Q4_0/with_silu", {Tensor::F32({1, 32}, xBasic), q4w},
                   DenseFn(GGMLQuantType::Q4_0, false, {activation::TypeSilu}), {{1.7616f, 2.8577f}}, 1e-3);
    RunTestGraphFn(b, "QuantizedDense_GGML_IQ4NL/basic", {Tensor::F32({1, 32}, xBasic), iqw}, DenseFn(GGMLQuantType::IQ4NL, false), {{14.f, 28.f}}, 1e-4);
    // Leading batch axes are flattened and restored: [2, 1, 32] -> [2, 1, 2].
    RunTestGraphFn(b, "QuantizedDense_GGML_Q8_0/rank3", {Tensor::F32({2, 1, 32}, xBatch), q8w}, DenseFn(GGMLQuantType::Q8_0, false),
                   {{2.f, 3.f, 1.f, 0.f}}, 1e-4);
}

static void TestQuantizedGather(Backend *b) {
    auto gatherFn = [](GGMLQuantType t) {
        return GraphFn([=](Function *f, const std::vector<Value> &in) {
            Quantization q = GGML(t);
            auto r = nn::QuantizedGather(f, in[0], in[1], &q);
            return std::make_pair(std::vector<Value>{r.first}, r.second);
        });
    };
    auto cat2 = [](std::vector<float> a, const std::vector<float> &c) { a.insert(a.end(), c.begin(), c.end()); return a; };
    const auto q8t = Tensor::U8({3, 34}, Cat({Q8Row(0x40, {0}), Q8Row(0x42, {1}), Q8Row(0x3C, {0, 1})}));
    const auto q4t = Tensor::U8({2, 18}, Cat({Q4Row(0x40, 0), Q4Row(0x42, 1)}));
    const auto iqt = Tensor::U8({2, 18}, Cat({Q4Row(0x3C, 0), Q4Row(0x40, 1)}));
    RunTestGraphFn(b, "QuantizedGather_Q8_0/basic", {q8t, Tensor::I32({2, 1}, {2, 0})}, gatherFn(GGMLQuantType::Q8_0),
                   {cat2(Unit({{0, 1.f}, {1, 1.f}}), Unit({{0, 2.f}}))}, 1e-4);
    RunTestGraphFn(b, "QuantizedGather_Q8_0/single", {q8t, Tensor::I32({1, 1}, {1})}, gatherFn(GGMLQuantType::Q8_0), {Unit({{1, 3.f}})}, 1e-4);
    RunTestGraphFn(b, "QuantizedGather_Q4_0/basic", {q4t, Tensor::I32({2, 1}, {1, 0})}, gatherFn(GGMLQuantType::Q4_0),
                   {cat2(Unit({{1, 3.f}}), Unit({{0, 2.f}}))}, 1e-4);
    // IQ4_NL code 8 decodes to +1, so the untouched positions are 1 * d, and code 9 to 13.
    std::vector<float> iqWant(32, 1.f);
    iqWant[0] = 13.f;
    RunTestGraphFn(b, "QuantizedGather_IQ4NL/basic", {iqt, Tensor::I32({1, 1}, {0})}, gatherFn(GGMLQuantType::IQ4NL), {iqWant}, 1e-4);

    // An index outside the table is an error of Execute, not a silent row.
    g_case = "QuantizedGather/out_of_range"; g_run++;
    auto builder = b->Builder(g_case);
    auto t = builder->Main()->Parameter("t", q8t.shape);
    auto i = builder->Main()->Parameter("i", Shape{DType::Int32, {1, 1}});
    Quantization q = GGML(GGMLQuantType::Q8_0);
    auto r = nn::QuantizedGather(builder->Main(), t.first, i.first, &q);
    CHECK(r.second.ok(), "%s", r.second.message.c_str());
    builder->Main()->Return({r.first});
    auto exec = builder->Compile();
    CHECK(exec.second.ok(), "%s", exec.second.message.c_str());
    int32_t bad = 3;
    auto tb = b->BufferFromFlatData(0, q8t.bytes.data(), q8t.shape);
    auto ib = b->BufferFromFlatData(0, &bad, Shape{DType::Int32, {1, 1}});
    auto res = exec.first->Execute({tb.first, ib.first});
    CHECK(!res.second.ok() && res.second.status == GQ_ERR_INVALID, "out-of-range index was accepted");
    std::printf("  ok   %s\n", g_case.c_str());
}

// One graph with independent projections (q/k/v) feeding nothing and a chained pair
// (gate -> down): independent nodes are submitted together, dependent ones in order.
static void TestLayerGraph(Backend *b) {
    const int K = 64, N = 64;
    // Q8_0 rows with d = 2^-3 (0x3000) and small integer codes; the expected values are
    // computed here in double from the same codes.
    auto makeW = [&](int seed, std::vector<double> &dense) {
        std::vector<uint8_t> w;
        dense.assign((size_t)N * K, 0.0);
        for (int n = 0; n < N; n++)
            for (int blk = 0; blk < K / 32; blk++) {
                w.push_back(0x00); w.push_back(0x30);
                for (int i = 0; i < 32; i++) {
                    int8_t q = (int8_t)(((n * 7 + blk * 13 + i * 3 + seed) % 9) - 4);
                    w.push_back((uint8_t)q);
                    dense[(size_t)n * K + blk * 32 + i] = q * 0.125;
                }
            }
        return w;
    };
    std::vector<double> dq, dk, dg, dd;
    auto wq = makeW(1, dq), wk = makeW(2, dk), wg = makeW(3, dg), wd = makeW(4, dd);
    std::vector<float> x((size_t)K);
    for (int i = 0; i < K; i++) x[(size_t)i] = (float)((i % 5) - 2) * 0.25f;
    auto matvec = [&](const std::vector<double> &w, const std::vector<double> &v, bool relu) {
        std::vector<double> y((size_t)N);
        for (int n = 0; n < N; n++) {
            double s = 0;
            for (int k = 0; k < K; k++) s += w[(size_t)n * K + k] * v[(size_t)k];
            y[(size_t)n] = relu && s < 0 ? 0 : s;
        }
        return y;
    };
    std::vector<double> xd(x.begin(), x.end());
    auto yq = matvec(dq, xd, false), yk = matvec(dk, xd, false), yg = matvec(dg, xd, true);
    // The chained input is the fp32 output of the first op.
    std::vector<double> yg32(yg.size());
    for (size_t i = 0; i < yg.size(); i++) yg32[i] = (double)(float)yg[i];
    auto ydn = matvec(dd, yg32, false);
    auto f32 = [](const std::vector<double> &v) { return std::vector<float>(v.begin(), v.end()); };
    GraphFn fn = [](Function *f, const std::vector<Value> &in) {
        Quantization q = GGML(GGMLQuantType::Q8_0);
        auto a = nn::QuantizedDense(f, in[0], in[1], &q, Value());
        auto c = nn::QuantizedDense(f, in[0], in[2], &q, Value());
        auto g = nn::QuantizedDense(f, in[0], in[3], &q, Value(), {activation::TypeRelu});
        if (!a.second.ok()) return std::make_pair(std::vector<Value>{}, a.second);
        if (!c.second.ok()) return std::make_pair(std::vector<Value>{}, c.second);
        if (!g.second.ok()) return std::make_pair(std::vector<Value>{}, g.second);
        auto d = nn::QuantizedDense(f, g.first, in[4], &q, Value());
        return std::make_pair(std::vector<Value>{a.first, c.first, d.first}, d.second);
    };
    RunTestGraphFn(b, "LayerGraph/independent_and_chained",
                   {Tensor::F32({1, K}, x), Tensor::U8({N, 68}, wq), Tensor::U8({N, 68}, wk), Tensor::U8({N, 68}, wg), Tensor::U8({N, 68}, wd)}, fn,
                   {f32(yq), f32(yk), f32(ydn)}, 1e-3);
}

static void TestExecuteArgumentErrors(Backend *b) {
    g_case = "Execute/argument_errors"; g_run++;
    auto builder = b->Builder(g_case);
    auto x = builder->Main()->Parameter("x", Shape{DType::Float32, {1, 32}});
    auto w = builder->Main()->Parameter("w", Shape{DType::Uint8, {2, 34}});
    Quantization q = GGML(GGMLQuantType::Q8_0);
    auto y = nn::QuantizedDense(builder->Main(), x.first, w.first, &q, Value());
    CHECK(y.second.ok(), "%s", y.second.message.c_str());
    auto shape = builder->OpShape(y.first);
    CHECK(shape.second.ok() && shape.first.dims == std::vector<int64_t>({1, 2}) && shape.first.dtype == DType::Float32, "OpShape is not Float32 [1, 2]");
    builder->Main()->Return({y.first});
    auto exec = builder->Compile();
    CHECK(exec.second.ok(), "%s", exec.second.message.c_str());
    std::vector<float> xv(32, 1.f);
    auto xb = b->BufferFromFlatData(0, xv.data(), Shape{DType::Float32, {1, 32}});
    CHECK(xb.second.ok(), "%s", xb.second.message.c_str());
    auto r1 = exec.first->Execute({xb.first});
    CHECK(!r1.second.ok() && r1.second.status == GQ_ERR_INVALID, "a missing input was accepted");
    auto r2 = exec.first->Execute({xb.first, xb.first});
    CHECK(!r2.second.ok() && r2.second.status == GQ_ERR_INVALID, "an input of the wrong shape was accepted");
    std::printf("  ok   %s\n", g_case.c_str());
}

// ---- graph-build validation and fallback rules: no GPU needed ------------------------------------
static void TestBuildTimeErrors() {
    g_case = "FusedQuantizedDense/build_time_errors"; g_run++;
    Function f;
    auto x = f.Parameter("x", Shape{DType::Float32, {1, 32}}).first;
    auto w = f.Parameter("w", Shape{DType::Uint8, {2, 34}}).first;
    auto wf = f.Parameter("wf", Shape{DType::Float32, {2, 34}}).first;
    auto bias3 = f.Parameter("b", Shape{DType::Float32, {3}}).first;
    auto xi = f.Parameter("xi", Shape{DType::Int32, {1, 32}}).first;
    Quantization q8 = GGML(GGMLQuantType::Q8_0), q4 = GGML(GGMLQuantType::Q4_0), q5k = GGML(GGMLQuantType(13)), q4k = GGML(GGMLQuantType::Q4_K);
    Quantization lin; lin.scheme = QuantScheme::Linear;
    // nil wq is a hard error (core/graph/fused_ops.go:198-200)
    auto r = f.FusedQuantizedDense(x, w, Value(), nullptr, ActivationType::None);
    CHECK(r.second.status == GQ_ERR_INVALID, "nil wq: status %d", r.second.status);
    // schemes and types outside the backend are "not implemented": the caller may fall back
    r = f.FusedQuantizedDense(x, w, Value(), &lin, ActivationType::None);
    CHECK(IsNotImplemented(r.second), "Linear scheme: status %d", r.second.status);
    r = f.FusedQuantizedDense(x, w, Value(), &q5k, ActivationType::None);
    CHECK(IsNotImplemented(r.second), "GGML type 13 (Q5_K): status %d", r.second.status);
    r = f.FusedQuantizedDense(xi, w, Value(), &q8, ActivationType::None);
    CHECK(IsNotImplemented(r.second), "Int32 activations: status %d", r.second.status);
    // malformed operands are hard errors
    r = f.FusedQuantizedDense(x, wf, Value(), &q8, ActivationType::None);
    CHECK(r.second.status == GQ_ERR_INVALID, "Float32 weights: status %d", r.second.status);
    r = f.FusedQuantizedDense(x, w, Value(), &q4, ActivationType::None);  // 34 is not a multiple of 18
    CHECK(r.second.status == GQ_ERR_INVALID, "ragged Q4_0 row: status %d", r.second.status);
    r = f.FusedQuantizedDense(x, w, bias3, &q8, ActivationType::None);
    CHECK(r.second.status == GQ_ERR_INVALID, "bias of wrong length: status %d", r.second.status);
    r = f.FusedQuantizedDense(x, w, Value(), &q4k, ActivationType::None);  // 34 bytes is not a Q4_K row
    CHECK(r.second.status == GQ_ERR_INVALID, "Q4_K row of 34 bytes: status %d", r.second.status);
    // more than one optional activation (ml/nn/quantized_dense.go:33-35)
    auto n = nn::QuantizedDense(&f, x, w, &q8, Value(), {activation::TypeRelu, activation::TypeTanh});
    CHECK(n.second.status == GQ_ERR_INVALID, "two activations: status %d", n.second.status);
    // the good case records the node and reports its shape
    r = f.FusedQuantizedDense(x, w, Value(), &q8, ActivationType::Gelu);
    CHECK(r.second.ok() && f.nodes()[(size_t)r.first.id].shape.dims == std::vector<int64_t>({1, 2}), "valid op rejected: %s", r.second.message.c_str());
    // gather validation
    auto idxBad = f.Parameter("i", Shape{DType::Int32, {2, 2}}).first;
    auto g = f.QuantizedEmbeddingLookup(w, idxBad, &q8);
    CHECK(g.second.status == GQ_ERR_INVALID, "indices [2,2]: status %d", g.second.status);
    auto gn = nn::QuantizedGather(&f, w, idxBad, &lin);
    CHECK(gn.second.status == GQ_ERR_INVALID, "gather with Linear scheme: status %d", gn.second.status);
    std::printf("  ok   %s\n", g_case.c_str());
}

static void TestFusedOpCaller() {
    g_case = "InternalFusedOpCaller/fallback_rules"; g_run++;
    Function f;
    auto x = f.Parameter("x", Shape{DType::Float32, {1, 32}}).first;
    auto w = f.Parameter("w", Shape{DType::Uint8, {2, 34}}).first;
    int fusedCalls = 0, decompCalls = 0;
    nn::NodeFn ok = [&]() { fusedCalls++; return std::make_pair(x, Error::None()); };
    nn::NodeFn notImpl = [&]() { fusedCalls++; return std::make_pair(Value(), Error::Make(GQ_ERR_NOT_IMPLEMENTED, "n/i")); };
    nn::NodeFn hard = [&]() { fusedCalls++; return std::make_pair(Value(), Error::Make(GQ_ERR_INVALID, "boom")); };
    nn::NodeFn decomp = [&]() { decompCalls++; return std::make_pair(w, Error::None()); };
    unsetenv("GOMLX_FUSION");
    bool fused = false;
    auto r = nn::InternalFusedOpCaller(ok, decomp, &fused);
    CHECK(r.second.ok() && r.first.id == x.id && fused && decompCalls == 0, "fused result was not used");
    r = nn::InternalFusedOpCaller(notImpl, decomp, &fused);
    CHECK(r.second.ok() && r.first.id == w.id && !fused && decompCalls == 1, "NotImplemented did not select the decomposed path");
    r = nn::InternalFusedOpCaller(hard, decomp, &fused);
    CHECK(r.second.status == GQ_ERR_INVALID && decompCalls == 1, "a hard error was masked by the fallback");
    setenv("GOMLX_FUSION", "0", 1);
    fusedCalls = 0;
    r = nn::InternalFusedOpCaller(ok, decomp, &fused);
    CHECK(r.second.ok() && r.first.id == w.id && fusedCalls == 0 && decompCalls == 2, "GOMLX_FUSION=0 still called the fused op");
    // Types without a decomposition ignore GOMLX_FUSION (ml/nn/quantized_dense.go:56).
    auto wk = f.Parameter("wk", Shape{DType::Uint8, {2, 144}}).first;
    auto xk = f.Parameter("xk", Shape{DType::Float32, {1, 256}}).first;
    Quantization q4k = GGML(GGMLQuantType::Q4_K), q8 = GGML(GGMLQuantType::Q8_0);
    auto n = nn::QuantizedDense(&f, xk, wk, &q4k, Value());
    CHECK(n.second.ok(), "Q4_K with GOMLX_FUSION=0: %s", n.second.message.c_str());
    // Decomposable types with fusion disabled and no general-purpose backend attached fail loudly.
    n = nn::QuantizedDense(&f, x, w, &q8, Value());
    CHECK(IsNotImplemented(n.second), "Q8_0 with GOMLX_FUSION=0 and no fallback: status %d", n.second.status);
    unsetenv("GOMLX_FUSION");
    n = nn::QuantizedDense(&f, x, w, &q8, Value());
    CHECK(n.second.ok(), "Q8_0 fused: %s", n.second.message.c_str());
    // ToBackend quirks (ml/layers/activation/activation.go:58-75)
    CHECK(activation::ToBackend(activation::TypeGeluApprox) == ActivationType::Gelu && activation::ToBackend(activation::TypeSwish) == ActivationType::Silu &&
              activation::ToBackend(activation::TypeSigmoid) == ActivationType::None && activation::ToBackend(activation::TypeSwiGLU) == ActivationType::None,
          "ToBackend mapping");
    std::printf("  ok   %s\n", g_case.c_str());
}

int main(int argc, char **argv) {
    const bool buildOnly = argc > 1 && std::string(argv[1]) == "--build-only";
    TestBuildTimeErrors();
    TestFusedOpCaller();
    if (!buildOnly) {
        auto backend = Backend::New(0);
        if (!backend.second.ok()) {
            std::printf("FAIL: no backend: %s\n", backend.second.message.c_str());
            return 2;
        }
        std::printf("backend: %s\n", backend.first->Description().c_str());
        TestQuantizedDenseGGML(backend.first.get());
        TestQuantizedGather(backend.first.get());
        TestLayerGraph(backend.first.get());
        TestExecuteArgumentErrors(backend.first.get());
    }
    std::printf("%d cases, %d failed\n", g_run, g_failed);
    return g_failed ? 1 : 0;
}
