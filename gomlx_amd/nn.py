"""Host-side mirror of the reference's quantized-Dense operator interface over torch
device tensors.  Names, argument meaning and error behaviour follow

* ``nn.QuantizedDense``   ml/nn/quantized_dense.go:31-57
* ``nn.QuantizedGather``  ml/nn/quantized_gather.go:30-43
* ``ggml.Dequantize``     ml/ggml/dequant.go:39-54
* ``graph.Quantization``  core/graph/fused_ops.go:18-48
* ``activation.Type.ToBackend``  ml/layers/activation/activation.go:58-75

torch only supplies device memory and the current stream; all arithmetic runs in
libgomlx_hipq.so.  There is no CPU path: tensors must live on the GPU.
"""
from __future__ import annotations

import enum
from dataclasses import dataclass

import torch

from . import _lib, ggml


class QuantizationScheme(enum.IntEnum):
    """compute.QuantizationScheme; only GGML is on this path."""
    LINEAR = 0
    NF4 = 1
    GGML = 2


class Activation(enum.IntEnum):
    """activation.Type of the reference (ml/layers/activation/activation.go:30-54)."""
    NONE = 0
    RELU = 1
    SIGMOID = 2
    HARD_SIGMOID = 3
    LEAKY_RELU = 4
    SELU = 5
    SWISH = 6
    HARD_SWISH = 7
    SILU = 8
    TANH = 9
    GELU = 10
    GELU_APPROX = 11
    SWIGLU = 12

    def to_backend(self) -> int:
        """activation.Type.ToBackend: types without a backend enum map to NONE, and both
        GELU flavours map to the single backend Gelu (activation.go:58-75)."""
        return {
            Activation.NONE: 0, Activation.GELU: 1, Activation.GELU_APPROX: 1, Activation.RELU: 2,
            Activation.SWISH: 3, Activation.SILU: 3, Activation.HARD_SWISH: 4, Activation.TANH: 5,
        }.get(self, 0)


@dataclass
class Quantization:
    """graph.Quantization (core/graph/fused_ops.go:18-48).  For GGML only scheme and
    ggml_type are used; the scales live inside the blocks."""
    scheme: QuantizationScheme = QuantizationScheme.GGML
    ggml_type: int = ggml.Q8_0
    scale: object = None
    zero_point: object = None
    block_axis: int = 0
    block_size: int = 0


def _stream_ptr(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_cuda(name: str, t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor: this backend has no CPU path")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _weights_2d(weights: torch.Tensor) -> None:
    if weights.dtype != torch.uint8 or weights.dim() != 2:
        raise ValueError("weights must be a Uint8 [N, bytesPerRow] tensor of native GGML blocks")


def dequantize(weights: torch.Tensor, ggml_type: int) -> torch.Tensor:
    """ggml.Dequantize: [N, bytesPerRow] uint8 -> [N, K] float32, bit-exact."""
    _require_cuda("weights", weights)
    _weights_2d(weights)
    _lib.init(weights.device.index or 0)
    N, rb = weights.shape
    bpb = ggml.bytes_per_block(ggml_type)
    if rb % bpb:
        raise ValueError(f"row of {rb} bytes is not a whole number of {bpb}-byte blocks")
    K = rb // bpb * ggml.values_per_block(ggml_type)
    out = torch.empty((N, K), dtype=torch.float32, device=weights.device)
    _lib.check(_lib.lib().gq_dequantize(ggml_type, weights.data_ptr(), N, K, out.data_ptr(), _stream_ptr(weights)))
    return out


@dataclass
class RMSNorm:
    """Configuration of norm.RMSNorm over the last axis (ml/layers/norm/rmsnorm.go:38-76): ``gain`` is the
    learned scale [K] (None = WithScale(false)), ``epsilon`` WithEpsilon (default 1e-6), ``scale_offset``
    WithScaleOffset (Gemma adds 1.0 to the scale)."""
    gain: torch.Tensor | None = None
    epsilon: float = 1e-6
    scale_offset: float = 0.0

    def _desc(self, K: int):
        if self.gain is not None:
            _require_cuda("gain", self.gain)
            if self.gain.dtype != torch.float32 or tuple(self.gain.shape) != (K,):
                raise ValueError(f"gain must be a float32 [{K}] tensor")
        return _lib.RmsNormDesc(None if self.gain is None else self.gain.data_ptr(), self.epsilon, self.scale_offset)


def rms_norm(x: torch.Tensor, norm: RMSNorm) -> torch.Tensor:
    """RMSNormBuilder.Done (ml/layers/norm/rmsnorm.go:78-113) over the last axis of a float32 tensor."""
    _require_cuda("x", x)
    if x.dtype != torch.float32:
        raise _lib.NotImplementedByBackend(_lib.ERR_NOT_IMPLEMENTED, f"rms_norm: dtype {x.dtype} is not implemented")
    K = x.shape[-1]
    d = norm._desc(K)
    _lib.init(x.device.index or 0)
    y = torch.empty_like(x)
    _lib.check(_lib.lib().gq_rmsnorm_f32(x.data_ptr(), x.numel() // K if K else 0, K, d.dGain, d.eps, d.gain_offset, y.data_ptr(),
                                         _stream_ptr(x)))
    return y


def gated_feed_forward(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, quant: Quantization, activation: Activation,
                       bias_gate: torch.Tensor | None = None, bias_up: torch.Tensor | None = None,
                       norm: RMSNorm | None = None) -> torch.Tensor:
    """The front of a gated feed-forward block (ml/zoo/transformer/transformer.go:1276-1287):
    ``activation(dense(xn, w_gate)) * dense(xn, w_up)`` with ``xn = rms_norm(x)`` when ``norm`` is given.
    x: [batch..., K] float32 or bfloat16 (gain, biases and the result stay float32); both weights [N, bytesPerRow] uint8 of one GGML type."""
    if quant is None or quant.scheme != QuantizationScheme.GGML:
        raise _lib.NotImplementedByBackend(_lib.ERR_NOT_IMPLEMENTED, "only the GGML scheme is on this path")
    for name, t in (("x", x), ("w_gate", w_gate), ("w_up", w_up)):
        _require_cuda(name, t)
    _weights_2d(w_gate)
    _weights_2d(w_up)
    if w_gate.shape != w_up.shape:
        raise ValueError(f"gate and up weights differ in shape: {tuple(w_gate.shape)} vs {tuple(w_up.shape)}")
    if x.dtype not in (torch.float32, torch.bfloat16):
        raise _lib.NotImplementedByBackend(_lib.ERR_NOT_IMPLEMENTED, f"gated_feed_forward: dtype {x.dtype} is not implemented")
    xd = _lib.F32 if x.dtype == torch.float32 else _lib.BF16
    import ctypes
    L = _lib.lib()
    N, rb = w_gate.shape
    K_in = x.shape[-1]
    M = x.numel() // K_in if K_in else 0
    K = ctypes.c_int64(0)
    for b in (bias_gate, bias_up):
        blen = -1
        if b is not None:
            _require_cuda("bias", b)
            if b.dtype != torch.float32 or b.dim() != 1:
                raise ValueError("bias must be a float32 [N] tensor")
            blen = b.shape[0]
        _lib.check(L.gq_qdense_check(quant.ggml_type, xd, M, K_in, N, rb, blen, activation.to_backend(), ctypes.byref(K)))
    d = None if norm is None else norm._desc(K.value)
    _lib.init(x.device.index or 0)
    y = torch.empty(x.shape[:-1] + (N,), dtype=torch.float32, device=x.device)
    fn = L.gq_qdense_gated_f32 if xd == _lib.F32 else L.gq_qdense_gated_bf16
    _lib.check(fn(quant.ggml_type, x.data_ptr(), M, K.value, None if d is None else ctypes.byref(d),
                                     w_gate.data_ptr(), None if bias_gate is None else bias_gate.data_ptr(), w_up.data_ptr(),
                                     None if bias_up is None else bias_up.data_ptr(), N, activation.to_backend(), y.data_ptr(),
                                     _stream_ptr(x)))
    return y


def quantized_dense(x: torch.Tensor, weights: torch.Tensor, quant: Quantization, bias: torch.Tensor | None = None,
                    *optional_activation: Activation, norm: RMSNorm | None = None,
                    residual: torch.Tensor | None = None) -> torch.Tensor:
    """nn.QuantizedDense for the GGML scheme: y = activation(x @ dequant(weights)^T + bias).

    x: [batch..., K] float32 or bfloat16; weights: [N, bytesPerRow] uint8; bias: [N] float32.
    Returns [batch..., N] float32.  ``norm`` applies an RMS normalisation to x first and ``residual``
    ([batch..., N] float32) is added to the result (gain and residual are float32 also for bfloat16 x): Model.normalize followed by a
    projection and Add(residual, ...) after it, ml/zoo/transformer/transformer.go:1099-1101, 1045, 1055.
    """
    if len(optional_activation) > 1:
        raise ValueError(f"quantized_dense can only take one optional activation, got {optional_activation}")
    act = optional_activation[0] if optional_activation else Activation.NONE
    if quant is None:
        raise ValueError("quant must not be None")  # core/graph/fused_ops.go:198-200
    if quant.scheme != QuantizationScheme.GGML:
        raise _lib.NotImplementedByBackend(_lib.ERR_NOT_IMPLEMENTED,
                                           f"scheme {quant.scheme.name} is outside this backend (GGML only)")
    _require_cuda("x", x)
    _require_cuda("weights", weights)
    _weights_2d(weights)
    if x.dtype == torch.float32:
        xd = _lib.F32
    elif x.dtype == torch.bfloat16:
        xd = _lib.BF16
    else:
        raise _lib.NotImplementedByBackend(_lib.ERR_NOT_IMPLEMENTED, f"activation dtype {x.dtype} is not implemented")
    L = _lib.lib()
    N, rb = weights.shape
    K_in = x.shape[-1]
    M = x.numel() // K_in if K_in else 0
    blen = -1
    if bias is not None:
        _require_cuda("bias", bias)
        if bias.dtype != torch.float32 or bias.dim() != 1:
            raise ValueError("bias must be a float32 [N] tensor")
        blen = bias.shape[0]
    import ctypes
    K = ctypes.c_int64(0)
    _lib.check(L.gq_qdense_check(quant.ggml_type, xd, M, K_in, N, rb, blen, act.to_backend(), ctypes.byref(K)))
    _lib.init(x.device.index or 0)
    y = torch.empty(x.shape[:-1] + (N,), dtype=torch.float32, device=x.device)
    if norm is not None or residual is not None:
        d = None if norm is None else norm._desc(K.value)
        if residual is not None:
            _require_cuda("residual", residual)
            if residual.dtype != torch.float32 or tuple(residual.shape) != tuple(y.shape):
                raise ValueError(f"residual must be a float32 tensor of shape {tuple(y.shape)}")
        block = L.gq_qdense_block_f32 if xd == _lib.F32 else L.gq_qdense_block_bf16
        _lib.check(block(quant.ggml_type, x.data_ptr(), M, K.value, None if d is None else ctypes.byref(d),
                                         weights.data_ptr(), N, None if bias is None else bias.data_ptr(), act.to_backend(),
                                         None if residual is None else residual.data_ptr(), y.data_ptr(), _stream_ptr(x)))
        return y
    fn = L.gq_qdense_f32 if xd == _lib.F32 else L.gq_qdense_bf16
    _lib.check(fn(quant.ggml_type, x.data_ptr(), M, K.value, weights.data_ptr(), N,
                  None if bias is None else bias.data_ptr(), act.to_backend(), y.data_ptr(), _stream_ptr(x)))
    return y


def quantized_gather(table: torch.Tensor, indices: torch.Tensor, quant: Quantization) -> torch.Tensor:
    """nn.QuantizedGather: indices [batch..., 1] (int32) -> [batch..., K] float32 rows of the
    dequantised table.  An out-of-range index raises IndexError."""
    if quant.scheme != QuantizationScheme.GGML:
        raise ValueError("quantized_gather: only the GGML scheme is supported")  # quantized_gather.go:31-33
    _require_cuda("table", table)
    _require_cuda("indices", indices)
    _weights_2d(table)
    if indices.dim() < 1 or indices.shape[-1] != 1:
        raise ValueError("indices must have last dimension 1")
    idx = indices.to(torch.int32).contiguous()
    _lib.init(table.device.index or 0)
    vocab, rb = table.shape
    bpb = ggml.bytes_per_block(quant.ggml_type)
    if rb % bpb:
        raise ValueError(f"row of {rb} bytes is not a whole number of {bpb}-byte blocks")
    K = rb // bpb * ggml.values_per_block(quant.ggml_type)
    count = idx.numel()
    out = torch.empty(tuple(indices.shape[:-1]) + (K,), dtype=torch.float32, device=table.device)
    flag = torch.zeros(1, dtype=torch.int32, device=table.device)
    _lib.check(_lib.lib().gq_embedding_lookup(quant.ggml_type, table.data_ptr(), vocab, K, idx.data_ptr(), count,
                                              out.data_ptr(), flag.data_ptr(), _stream_ptr(table)))
    if count and int(flag.item()):
        raise IndexError("quantized_gather: index out of range")
    return out


def quantized_dense_batch(problems, norm: RMSNorm | None = None) -> list:
    """Several independent nn.QuantizedDense calls submitted together (gq_qdense_f32_batch); with
    ``norm`` every problem's activations are RMS-normalised first (the q/k/v projections behind a
    layer's input norm, gq_qdense_norm_f32_batch).

    ``problems`` is a sequence of ``(x, weights, quant, bias, activation)`` tuples with float32
    activations (with ``norm``: all float32 or all bfloat16); returns the list of outputs.  Results equal those of separate calls; problems
    of one GGML type and one batch size of up to 8 rows share a single kernel launch.
    """
    import ctypes
    L = _lib.lib()
    descs = (_lib.DenseDesc * len(problems))()
    outs = []
    for i, (x, weights, quant, bias, act) in enumerate(problems):
        act = Activation.NONE if act is None else act
        if quant is None or quant.scheme != QuantizationScheme.GGML:
            raise _lib.NotImplementedByBackend(_lib.ERR_NOT_IMPLEMENTED, "only the GGML scheme is on this path")
        _require_cuda("x", x)
        _require_cuda("weights", weights)
        _weights_2d(weights)
        bf16 = norm is not None and x.dtype == torch.bfloat16 and all(p[0].dtype == torch.bfloat16 for p in problems)
        if x.dtype != torch.float32 and not bf16:
            raise _lib.NotImplementedByBackend(_lib.ERR_NOT_IMPLEMENTED, "batched submission takes float32 activations "
                                               "(behind a shared normalisation: all float32 or all bfloat16)")
        N, rb = weights.shape
        K_in = x.shape[-1]
        M = x.numel() // K_in if K_in else 0
        blen = -1
        if bias is not None:
            _require_cuda("bias", bias)
            blen = bias.shape[0]
        K = ctypes.c_int64(0)
        _lib.check(L.gq_qdense_check(quant.ggml_type, _lib.BF16 if bf16 else _lib.F32, M, K_in, N, rb, blen, act.to_backend(), ctypes.byref(K)))
        y = torch.empty(x.shape[:-1] + (N,), dtype=torch.float32, device=x.device)
        outs.append(y)
        d = descs[i]
        d.type, d.act, d.dX, d.M, d.K = quant.ggml_type, act.to_backend(), x.data_ptr(), M, K.value
        d.dW, d.N, d.dBias, d.dY = weights.data_ptr(), N, (None if bias is None else bias.data_ptr()), y.data_ptr()
    if problems:
        _lib.init(problems[0][0].device.index or 0)
        if norm is None:
            _lib.check(L.gq_qdense_f32_batch(len(problems), descs, _stream_ptr(problems[0][0])))
        else:
            d = norm._desc(problems[0][0].shape[-1])
            fn = L.gq_qdense_norm_bf16_batch if problems[0][0].dtype == torch.bfloat16 else L.gq_qdense_norm_f32_batch
            _lib.check(fn(len(problems), descs, ctypes.byref(d), _stream_ptr(problems[0][0])))
    return outs
