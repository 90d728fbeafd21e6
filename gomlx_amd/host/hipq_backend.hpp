// Host-side mirror, in C++, of the part of GoMLX's backend interface that the quantized Dense
// path goes through.  GoMLX is Go and its backends implement the interfaces of
// github.com/gomlx/compute (Backend / Builder / Function / Executable / Buffer); no Go toolchain
// is available to this build, so the same operator surface is written in C++ directly above
// the C ABI of libgomlx_hipq.so.  Names, argument meaning and error behaviour follow the
// reference call sites:
//
//   compute.Backend         core/tensors/ondevice.go:273-285 (BufferFromFlatData), :462 (ToFlatData)
//   compute.Builder         core/graph/graph.go:277 (Builder), :498 (Compile); fused_ops.go:238 (OpShape)
//   compute.Function        core/graph/fused_ops.go:231-232 (FusedQuantizedDense), :295-296 (QuantizedEmbeddingLookup)
//   compute.Executable      core/graph/graph.go:669 (Execute)
//   nn.QuantizedDense       ml/nn/quantized_dense.go:31-57
//   nn.QuantizedGather      ml/nn/quantized_gather.go:30-43
//   InternalFusedOpCaller   core/graph/fused_ops.go:339-373 (GOMLX_FUSION, NotImplemented fallback)
//
// Only the hot ops are implemented natively; every other op reports ErrNotImplemented, which
// is what makes a wrapping Go backend delegate it to the general-purpose backend.
// Errors are returned, never thrown: `Error::ok()` / `IsNotImplemented(err)`.
#pragma once

#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "../../include/gomlx_hipq.h"

namespace gomlx_hipq {

// ---- errors ---------------------------------------------------------------------------------
struct Error {
    int status = GQ_OK;
    std::string message;
    bool ok() const { return status == GQ_OK; }
    static Error None() { return Error(); }
    static Error Make(int status, std::string msg) { Error e; e.status = status; e.message = std::move(msg); return e; }
    static Error FromLast(int status) { return Make(status, gq_last_error()); }
};
// compute.IsNotImplemented(err): the caller may fall back to a decomposed graph.
inline bool IsNotImplemented(const Error &e) { return e.status == GQ_ERR_NOT_IMPLEMENTED; }

// ---- dtypes / shapes ------------------------------------------------------------------------
enum class DType { Float32, BFloat16, Uint8, Int32 };
inline size_t SizeOf(DType t) { return t == DType::Float32 || t == DType::Int32 ? 4 : (t == DType::BFloat16 ? 2 : 1); }
struct Shape {
    DType dtype = DType::Float32;
    std::vector<int64_t> dims;
    int64_t Size() const { int64_t n = 1; for (int64_t d : dims) n *= d; return n; }
    int Rank() const { return (int)dims.size(); }
    bool operator==(const Shape &o) const { return dtype == o.dtype && dims == o.dims; }
};

// compute.QuantizationScheme / GGMLQuantType / ActivationType
enum class QuantScheme { Linear, NF4, GGML };
enum class GGMLQuantType { Q4_0 = GQ_Q4_0, Q8_0 = GQ_Q8_0, Q4_K = GQ_Q4_K, Q6_K = GQ_Q6_K, IQ4NL = GQ_IQ4_NL };
inline int BytesPerBlock(GGMLQuantType t) { return gq_bytes_per_block((int)t); }
inline int ValuesPerBlock(GGMLQuantType t) { return gq_values_per_block((int)t); }
enum class ActivationType { None = GQ_ACT_NONE, Gelu = GQ_ACT_GELU, Relu = GQ_ACT_RELU, Silu = GQ_ACT_SILU,
                            HardSwish = GQ_ACT_HARDSWISH, Tanh = GQ_ACT_TANH };

// activation.Type and its ToBackend mapping (ml/layers/activation/activation.go:30-75)
namespace activation {
enum Type { TypeNone, TypeRelu, TypeSigmoid, TypeHardSigmoid, TypeLeakyRelu, TypeSelu, TypeSwish, TypeHardSwish, TypeSilu,
            TypeTanh, TypeGelu, TypeGeluApprox, TypeSwiGLU };
inline ActivationType ToBackend(Type t) {
    switch (t) {
    case TypeGelu: case TypeGeluApprox: return ActivationType::Gelu;
    case TypeRelu: return ActivationType::Relu;
    case TypeSwish: case TypeSilu: return ActivationType::Silu;
    case TypeHardSwish: return ActivationType::HardSwish;
    case TypeTanh: return ActivationType::Tanh;
    default: return ActivationType::None;  // unsupported types map to None (activation.go:72-73)
    }
}
}  // namespace activation

class Backend;

// ---- compute.Buffer -------------------------------------------------------------------------
class Buffer {
public:
    Buffer(Backend *b, Shape s, void *dptr) : backend_(b), shape_(std::move(s)), dptr_(dptr) {}
    ~Buffer() { Finalize(); }
    Buffer(const Buffer &) = delete;
    Buffer &operator=(const Buffer &) = delete;
    const Shape &GetShape() const { return shape_; }
    Backend *GetBackend() const { return backend_; }
    int DeviceNum() const { return 0; }
    void *DevicePtr() const { return dptr_; }
    Error ToFlatData(void *flat) const {  // device -> host, returns when the copy is done
        if (!dptr_ && shape_.Size() > 0) return Error::Make(GQ_ERR_INVALID, "buffer was finalized");
        int rc = gq_d2h(flat, dptr_, (size_t)shape_.Size() * SizeOf(shape_.dtype), nullptr);
        return rc ? Error::FromLast(rc) : Error::None();
    }
    void Finalize() { if (dptr_) { gq_free(dptr_); dptr_ = nullptr; } }
private:
    Backend *backend_;
    Shape shape_;
    void *dptr_;
};
using BufferPtr = std::shared_ptr<Buffer>;

// ---- graph under construction -----------------------------------------------------------------
struct Value { int id = -1; bool valid() const { return id >= 0; } };

struct Quantization {  // compute.Quantization (core/graph/fused_ops.go:53-65)
    QuantScheme scheme = QuantScheme::GGML;
    Value scale, zeroPoint;
    int blockAxis = 0, blockSize = 0;
    GGMLQuantType ggmlType = GGMLQuantType::Q8_0;
};

enum class OpKind { Parameter, FusedQuantizedDense, QuantizedEmbeddingLookup };
struct Node {
    OpKind kind;
    Shape shape;
    std::vector<int> inputs;  // node ids; for FusedQuantizedDense: x, weights, [bias]
    int param_index = -1;
    GGMLQuantType ggmlType = GGMLQuantType::Q8_0;
    ActivationType act = ActivationType::None;
    int64_t K = 0;
    bool has_bias = false;
};

class Executable;

// compute.Function: the op methods validate and record at graph-build time; kernels run in Execute.
class Function {
public:
    std::pair<Value, Error> Parameter(const std::string &name, const Shape &shape) {
        (void)name;
        Node n; n.kind = OpKind::Parameter; n.shape = shape; n.param_index = num_params_++;
        return {Push(n), Error::None()};
    }

    // FusedQuantizedDense(x, weights, bias, wq, activation) (core/graph/fused_ops.go:231-232).
    // bias may be an invalid Value (nil).  Unsupported -> ErrNotImplemented, malformed -> hard error.
    std::pair<Value, Error> FusedQuantizedDense(Value x, Value weights, Value bias, const Quantization *wq, ActivationType act) {
        if (!wq) return {Value(), Error::Make(GQ_ERR_INVALID, "FusedQuantizedDense: wq must not be nil")};
        if (wq->scheme != QuantScheme::GGML)
            return {Value(), Error::Make(GQ_ERR_NOT_IMPLEMENTED, "FusedQuantizedDense: only the GGML scheme is implemented by this backend")};
        if (!Known(x) || !Known(weights) || (bias.valid() && !Known(bias)))
            return {Value(), Error::Make(GQ_ERR_INVALID, "FusedQuantizedDense: operand does not belong to this function")};
        const Shape &xs = nodes_[x.id].shape, &ws = nodes_[weights.id].shape;
        if (ws.dtype != DType::Uint8 || ws.Rank() != 2)
            return {Value(), Error::Make(GQ_ERR_INVALID, "FusedQuantizedDense: GGML weights must be Uint8 [N, bytesPerRow]")};
        if (xs.Rank() < 1) return {Value(), Error::Make(GQ_ERR_INVALID, "FusedQuantizedDense: x must have rank >= 1")};
        int xd;
        if (xs.dtype == DType::Float32) xd = GQ_F32;
        else if (xs.dtype == DType::BFloat16) xd = GQ_BF16;
        else return {Value(), Error::Make(GQ_ERR_NOT_IMPLEMENTED, "FusedQuantizedDense: activation dtype is not implemented")};
        int64_t blen = -1;
        if (bias.valid()) {
            const Shape &bs = nodes_[bias.id].shape;
            if (bs.dtype != DType::Float32 || bs.Rank() != 1) return {Value(), Error::Make(GQ_ERR_INVALID, "FusedQuantizedDense: bias must be Float32 [N]")};
            blen = bs.dims[0];
        }
        const int64_t kin = xs.dims.back(), M = kin ? xs.Size() / kin : 0;
        int64_t K = 0;
        int rc = gq_qdense_check((int)wq->ggmlType, xd, M, kin, ws.dims[0], ws.dims[1], blen, (int)act, &K);
        if (rc) return {Value(), Error::FromLast(rc)};
        Node n; n.kind = OpKind::FusedQuantizedDense; n.ggmlType = wq->ggmlType; n.act = act; n.K = K; n.has_bias = bias.valid();
        n.shape.dtype = DType::Float32;
        n.shape.dims = xs.dims; n.shape.dims.back() = ws.dims[0];
        n.inputs = {x.id, weights.id};
        if (bias.valid()) n.inputs.push_back(bias.id);
        return {Push(n), Error::None()};
    }

    // QuantizedEmbeddingLookup(data, indices, tq) (core/graph/fused_ops.go:295-296); indices [..., 1] Int32.
    std::pair<Value, Error> QuantizedEmbeddingLookup(Value data, Value indices, const Quantization *tq) {
        if (!tq) return {Value(), Error::Make(GQ_ERR_INVALID, "QuantizedEmbeddingLookup: tq must not be nil")};
        if (tq->scheme != QuantScheme::GGML) return {Value(), Error::Make(GQ_ERR_INVALID, "QuantizedEmbeddingLookup: only QuantGGML is supported")};
        if (!Known(data) || !Known(indices)) return {Value(), Error::Make(GQ_ERR_INVALID, "QuantizedEmbeddingLookup: bad operand")};
        const Shape &ts = nodes_[data.id].shape, &is = nodes_[indices.id].shape;
        const int bpb = BytesPerBlock(tq->ggmlType);
        if (bpb == 0) return {Value(), Error::Make(GQ_ERR_NOT_IMPLEMENTED, "QuantizedEmbeddingLookup: GGML type is not implemented")};
        if (ts.dtype != DType::Uint8 || ts.Rank() != 2 || ts.dims[1] % bpb) return {Value(), Error::Make(GQ_ERR_INVALID, "QuantizedEmbeddingLookup: table must be Uint8 [vocab, bytesPerRow]")};
        if (is.dtype != DType::Int32 || is.Rank() < 1 || is.dims.back() != 1) return {Value(), Error::Make(GQ_ERR_INVALID, "QuantizedEmbeddingLookup: indices must be Int32 [..., 1]")};
        Node n; n.kind = OpKind::QuantizedEmbeddingLookup; n.ggmlType = tq->ggmlType;
        n.K = ts.dims[1] / bpb * ValuesPerBlock(tq->ggmlType);
        n.shape.dtype = DType::Float32;
        n.shape.dims.assign(is.dims.begin(), is.dims.end() - 1);
        n.shape.dims.push_back(n.K);
        n.inputs = {data.id, indices.id};
        return {Push(n), Error::None()};
    }

    // Any op outside the hot path: a wrapping backend delegates it (fused_ops.go:357-363).
    std::pair<Value, Error> NotImplementedOp(const char *name) {
        return {Value(), Error::Make(GQ_ERR_NOT_IMPLEMENTED, std::string(name) + ": not implemented by the hipq backend")};
    }

    Error Return(const std::vector<Value> &outputs) {
        for (Value v : outputs) if (!Known(v)) return Error::Make(GQ_ERR_INVALID, "Return: unknown value");
        outputs_ = outputs;
        return Error::None();
    }

    bool Known(Value v) const { return v.id >= 0 && v.id < (int)nodes_.size(); }
    const std::vector<Node> &nodes() const { return nodes_; }
    const std::vector<Value> &outputs() const { return outputs_; }
    int num_params() const { return num_params_; }
private:
    Value Push(const Node &n) { nodes_.push_back(n); Value v; v.id = (int)nodes_.size() - 1; return v; }
    std::vector<Node> nodes_;
    std::vector<Value> outputs_;
    int num_params_ = 0;
};

// ---- compute.Executable -----------------------------------------------------------------------
class Executable {
public:
    Executable(Backend *b, std::vector<Node> nodes, std::vector<Value> outputs, int nparams)
        : backend_(b), nodes_(std::move(nodes)), outputs_(std::move(outputs)), nparams_(nparams) {}

    // Execute(inputs, donate, defaultDevice) (core/graph/graph.go:669).  Nodes run in topological
    // "levels": FusedQuantizedDense nodes of one level have no dependencies among them and go out
    // as one batched submission.
    std::pair<std::vector<BufferPtr>, Error> Execute(const std::vector<BufferPtr> &inputs, const std::vector<bool> &donate = {},
                                                    int defaultDevice = 0);
private:
    Backend *backend_;
    std::vector<Node> nodes_;
    std::vector<Value> outputs_;
    int nparams_;
};

// ---- compute.Builder --------------------------------------------------------------------------
class Builder {
public:
    explicit Builder(Backend *b, std::string name) : backend_(b), name_(std::move(name)) {}
    Function *Main() { return &main_; }
    std::pair<Shape, Error> OpShape(Value v) const {
        if (!main_.Known(v)) return {Shape(), Error::Make(GQ_ERR_INVALID, "OpShape: unknown value")};
        return {main_.nodes()[v.id].shape, Error::None()};
    }
    std::pair<std::unique_ptr<Executable>, Error> Compile() {
        if (main_.outputs().empty()) return {nullptr, Error::Make(GQ_ERR_INVALID, "Compile: Main().Return() was not called")};
        return {std::unique_ptr<Executable>(new Executable(backend_, main_.nodes(), main_.outputs(), main_.num_params())), Error::None()};
    }
private:
    Backend *backend_;
    std::string name_;
    Function main_;
};

// ---- compute.Backend --------------------------------------------------------------------------
class Backend {
public:
    // compute.NewWithConfig("hipq[:device]"): fails when there is no gfx950 device.
    static std::pair<std::unique_ptr<Backend>, Error> New(int device = 0) {
        int rc = gq_init(device);
        if (rc) return {nullptr, Error::FromLast(rc)};
        return {std::unique_ptr<Backend>(new Backend()), Error::None()};
    }
    std::string Name() const { return "hipq"; }
    std::string Description() const { char b[256] = ""; gq_device_name(b, sizeof b); return std::string("gomlx_hipq on ") + b; }
    int NumDevices() const { return 1; }
    bool HasSharedBuffers() const { return false; }
    std::unique_ptr<gomlx_hipq::Builder> Builder(const std::string &name) { return std::unique_ptr<gomlx_hipq::Builder>(new gomlx_hipq::Builder(this, name)); }
    std::pair<BufferPtr, Error> BufferFromFlatData(int deviceNum, const void *flat, const Shape &shape) {
        if (deviceNum != 0) return {nullptr, Error::Make(GQ_ERR_INVALID, "BufferFromFlatData: this backend drives one device")};
        void *d = nullptr;
        const size_t bytes = (size_t)shape.Size() * SizeOf(shape.dtype);
        int rc = gq_malloc(&d, bytes);
        if (rc) return {nullptr, Error::FromLast(rc)};
        rc = gq_h2d(d, flat, bytes, nullptr);
        if (rc) { gq_free(d); return {nullptr, Error::FromLast(rc)}; }
        return {std::make_shared<Buffer>(this, shape, d), Error::None()};
    }
    std::pair<BufferPtr, Error> NewBuffer(const Shape &shape) {
        void *d = nullptr;
        int rc = gq_malloc(&d, (size_t)shape.Size() * SizeOf(shape.dtype));
        if (rc) return {nullptr, Error::FromLast(rc)};
        return {std::make_shared<Buffer>(this, shape, d), Error::None()};
    }
    void Finalize() {}
private:
    Backend() = default;
};

inline std::pair<std::vector<BufferPtr>, Error> Executable::Execute(const std::vector<BufferPtr> &inputs, const std::vector<bool> &donate,
                                                                    int defaultDevice) {
    (void)donate; (void)defaultDevice;
    std::vector<BufferPtr> none;
    if ((int)inputs.size() != nparams_)  // core/graph/graph.go:570-573
        return {none, Error::Make(GQ_ERR_INVALID, "Execute: expected " + std::to_string(nparams_) + " inputs, got " + std::to_string(inputs.size()))};
    std::vector<BufferPtr> val(nodes_.size());
    std::vector<int> level(nodes_.size(), 0);
    int max_level = 0;
    for (size_t i = 0; i < nodes_.size(); i++) {
        const Node &n = nodes_[i];
        if (n.kind == OpKind::Parameter) {
            const BufferPtr &b = inputs[n.param_index];
            if (!b || (!b->DevicePtr() && b->GetShape().Size() > 0)) return {none, Error::Make(GQ_ERR_INVALID, "Execute: input buffer is nil or finalized")};
            if (!(b->GetShape() == n.shape)) return {none, Error::Make(GQ_ERR_INVALID, "Execute: input shape differs from the parameter's")};
            val[i] = b;
        } else {
            for (int in : n.inputs) level[i] = level[i] > level[in] + 1 ? level[i] : level[in] + 1;
            if (level[i] > max_level) max_level = level[i];
        }
    }
    for (int lv = 1; lv <= max_level; lv++) {
        std::vector<gq_dense_desc> batch;
        for (size_t i = 0; i < nodes_.size(); i++) {
            const Node &n = nodes_[i];
            if (level[i] != lv || n.kind == OpKind::Parameter) continue;
            auto out = backend_->NewBuffer(n.shape);
            if (!out.second.ok()) return {none, out.second};
            val[i] = out.first;
            if (n.kind == OpKind::FusedQuantizedDense) {
                const Shape &xs = nodes_[n.inputs[0]].shape, &ws = nodes_[n.inputs[1]].shape;
                const int64_t M = n.K ? xs.Size() / n.K : 0;
                const void *bias = n.has_bias ? val[n.inputs[2]]->DevicePtr() : nullptr;
                if (xs.dtype == DType::Float32) {
                    gq_dense_desc d;
                    d.type = (int)n.ggmlType; d.act = (int)n.act; d.dX = (const float *)val[n.inputs[0]]->DevicePtr(); d.M = M; d.K = n.K;
                    d.dW = val[n.inputs[1]]->DevicePtr(); d.N = ws.dims[0]; d.dBias = (const float *)bias; d.dY = (float *)val[i]->DevicePtr();
                    batch.push_back(d);
                } else {
                    int rc = gq_qdense_bf16((int)n.ggmlType, (const uint16_t *)val[n.inputs[0]]->DevicePtr(), M, n.K, val[n.inputs[1]]->DevicePtr(),
                                            ws.dims[0], (const float *)bias, (int)n.act, (float *)val[i]->DevicePtr(), nullptr);
                    if (rc) return {none, Error::FromLast(rc)};
                }
            } else {  // QuantizedEmbeddingLookup
                const Shape &ts = nodes_[n.inputs[0]].shape, &is = nodes_[n.inputs[1]].shape;
                auto flag = backend_->NewBuffer(Shape{DType::Int32, {1}});
                if (!flag.second.ok()) return {none, flag.second};
                int32_t zero = 0;
                gq_h2d(flag.first->DevicePtr(), &zero, 4, nullptr);
                int rc = gq_embedding_lookup((int)n.ggmlType, val[n.inputs[0]]->DevicePtr(), ts.dims[0], n.K, (const int32_t *)val[n.inputs[1]]->DevicePtr(),
                                             is.Size(), (float *)val[i]->DevicePtr(), (int32_t *)flag.first->DevicePtr(), nullptr);
                if (rc) return {none, Error::FromLast(rc)};
                int32_t bad = 0;
                flag.first->ToFlatData(&bad);
                if (bad) return {none, Error::Make(GQ_ERR_INVALID, "QuantizedEmbeddingLookup: index out of range")};
            }
        }
        if (!batch.empty()) {
            int rc = gq_qdense_f32_batch((int)batch.size(), batch.data(), nullptr);
            if (rc) return {none, Error::FromLast(rc)};
        }
    }
    int rc = gq_sync(nullptr);
    if (rc) return {none, Error::FromLast(rc)};
    std::vector<BufferPtr> outs;
    for (Value v : outputs_) outs.push_back(val[v.id]);
    return {outs, Error::None()};
}

// ---- graph.Quantization + nn.* operator layer ---------------------------------------------------
namespace nn {

// InternalFusedOpCaller (core/graph/fused_ops.go:339-373): with GOMLX_FUSION disabled the fused op
// is never used; a NotImplemented error from `fused` selects `decomposed`; other errors surface.
inline bool FusionEnabled() {
    const char *e = std::getenv("GOMLX_FUSION");
    if (!e || !*e) return true;
    return !(std::strcmp(e, "0") == 0 || std::strcmp(e, "false") == 0 || std::strcmp(e, "False") == 0 || std::strcmp(e, "FALSE") == 0 ||
             std::strcmp(e, "f") == 0 || std::strcmp(e, "F") == 0);
}
using NodeFn = std::function<std::pair<Value, Error>()>;
inline std::pair<Value, Error> InternalFusedOpCaller(const NodeFn &fused, const NodeFn &decomposed, bool *opFused = nullptr) {
    if (opFused) *opFused = false;
    if (!FusionEnabled()) return decomposed();
    auto r = fused();
    if (r.second.ok()) { if (opFused) *opFused = true; return r; }
    if (IsNotImplemented(r.second)) return decomposed();
    return r;  // unexpected error: surfaces instead of being masked (fused_ops.go:365)
}

// ggml.CanDecompose (ml/ggml/dequant.go:20-27)
inline bool CanDecompose(GGMLQuantType t) { return t == GGMLQuantType::Q4_0 || t == GGMLQuantType::Q8_0 || t == GGMLQuantType::IQ4NL; }

// nn.QuantizedDense (ml/nn/quantized_dense.go:31-57), GGML branch.  `decomposed` stands for
// ggml.DenseDecomposed, which needs the general-purpose backend's primitives; pass nullptr when
// no such backend is attached (the call then fails if the fused op cannot be used).
inline std::pair<Value, Error> QuantizedDense(Function *f, Value x, Value weights, const Quantization *quant, Value bias,
                                              std::vector<activation::Type> optionalActivation = {}, const NodeFn &decomposed = nullptr) {
    if (optionalActivation.size() > 1)
        return {Value(), Error::Make(GQ_ERR_INVALID, "nn.QuantizedDense() can only take one optional activation")};
    const activation::Type act = optionalActivation.empty() ? activation::TypeNone : optionalActivation[0];
    if (!quant) return {Value(), Error::Make(GQ_ERR_INVALID, "BackendFusedQuantizedDense: wq must not be nil")};
    const ActivationType backendAct = activation::ToBackend(act);
    NodeFn fused = [&]() { return f->FusedQuantizedDense(x, weights, bias, quant, backendAct); };
    if (quant->scheme == QuantScheme::GGML && !CanDecompose(quant->ggmlType)) return fused();  // quantized_dense.go:56
    NodeFn fallback = decomposed ? decomposed : NodeFn([&]() {
        return std::make_pair(Value(), Error::Make(GQ_ERR_NOT_IMPLEMENTED, "nn.QuantizedDense: the decomposed path needs the general-purpose backend"));
    });
    return InternalFusedOpCaller(fused, fallback);
}

// nn.QuantizedGather (ml/nn/quantized_gather.go:30-43)
inline std::pair<Value, Error> QuantizedGather(Function *f, Value table, Value indices, const Quantization *quant,
                                               const NodeFn &decomposed = nullptr) {
    if (!quant || quant->scheme != QuantScheme::GGML)
        return {Value(), Error::Make(GQ_ERR_INVALID, "nn.QuantizedGather: only QuantGGML scheme is supported")};
    NodeFn fused = [&]() { return f->QuantizedEmbeddingLookup(table, indices, quant); };
    if (!CanDecompose(quant->ggmlType)) return fused();
    NodeFn fallback = decomposed ? decomposed : NodeFn([&]() {
        return std::make_pair(Value(), Error::Make(GQ_ERR_NOT_IMPLEMENTED, "nn.QuantizedGather: the decomposed path needs the general-purpose backend"));
    });
    return InternalFusedOpCaller(fused, fallback);
}

}  // namespace nn
}  // namespace gomlx_hipq
