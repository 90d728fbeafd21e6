"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares,
and its host-only entry points (geometry, build-time validation, error reporting) behave
like the reference's graph-build checks.  No kernel is launched here."""
import ctypes
import os
import re

import pytest

from gomlx_amd import _lib, ggml

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "gomlx_hipq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gq_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_all_exported_and_bound():
    syms = declared_symbols()
    assert len(syms) >= 20
    L = ctypes.CDLL(_lib.LIB_PATH)
    for s in syms:
        assert hasattr(L, s), f"{s} is declared in the header but not exported"
    bound = {name for name, _, _ in _lib.SIGNATURES}
    assert bound == set(syms)


def test_go_binding_source_names_only_what_the_header_declares():
    """The cgo source under go/hipbackend cannot be compiled here (no Go toolchain): at least every C name it uses
    must exist in the header - functions, the two structs and the constants."""
    text = open(os.path.join(ROOT, "include", "gomlx_hipq.h")).read()
    header_names = set(re.findall(r"\b(gq_[a-z0-9_]+|GQ_[A-Z0-9_]+)\b", re.sub(r"/\*.*?\*/", "", text, flags=re.S)))
    used = set()
    godir = os.path.join(ROOT, "go", "hipbackend")
    for fn in os.listdir(godir):
        if fn.endswith(".go"):
            used |= set(re.findall(r"\bC\.(gq_[a-z0-9_]+|GQ_[A-Z0-9_]+)\b", open(os.path.join(godir, fn)).read()))
    assert len(used) >= 15
    assert used <= header_names, sorted(used - header_names)
    # both fused ops of the path are bound
    assert {"gq_qdense_f32", "gq_qdense_bf16", "gq_embedding_lookup", "gq_qdense_check"} <= used


def test_ablation_variants_still_apply_to_the_sources():
    """The timing-only builds of the benchmark are made by exact text substitution on the kernel sources: every
    substitution must still find its text (a kernel edit that moves it has to move the variant too)."""
    from gomlx_amd import ablate
    for name in ablate.VARIANTS:
        assert ablate.variant_source(name)


def test_written_out_memory_instructions_keep_their_wait_states(tmp_path):
    """A vector-memory instruction that reads a scalar register needs five wait states after a vector instruction wrote
    that register (v_readfirstlane and friends).  The compiler inserts them for its own loads; for instructions written
    out as text it cannot, and a load that runs too early takes the register's previous contents as its address.  The
    GEMM's LDS-DMA copies are such text: its assembly must show no vector-ALU write to their scalar operands within the
    five instructions in front of them."""
    import subprocess
    from gomlx_amd import build as B
    asm = tmp_path / "gemm_dma.s"
    flags = [f for f in B.HIPCC_FLAGS if not f.startswith("-Rpass")]
    r = subprocess.run([B.hipcc(), *flags, "-S", "--cuda-device-only", "-I", B.CSRC, os.path.join(B.CSRC, "gemm_dma.hip"), "-o", str(asm)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = asm.read_text().split("\n")
    checked = 0
    for i, l in enumerate(lines):
        m = re.search(r"buffer_load_dwordx4 v\d+, s\[(\d+):(\d+)\], (s\d+) offen lds", l)
        if not m:
            continue
        checked += 1
        sregs = {f"s{k}" for k in range(int(m.group(1)), int(m.group(2)) + 1)} | {m.group(3)}
        k, seen = i - 1, 0
        while k > 0 and seen < 5:
            t = lines[k].strip()
            k -= 1
            if not t or t.startswith((";", ".")):
                continue
            seen += 1
            if t.startswith("v_") and t.split()[1].rstrip(",") in sregs:
                raise AssertionError(f"line {k + 2}: {t!r} writes a scalar operand of the copy at line {i + 1} {seen - 1} instructions before it")
    assert checked > 100  # every instance of the kernel carries its copies


def test_no_oracle_or_torch_linked_into_the_library():
    import subprocess
    out = subprocess.run(["ldd", _lib.LIB_PATH], capture_output=True, text=True).stdout
    assert "libamdhip64" in out
    assert "ggml_oracle" not in out and "torch" not in out


def test_no_kernel_spills_registers():
    """The build records every kernel's resource use; a kernel that needs scratch memory (register
    spills) runs far slower than designed, and the build refuses it."""
    import json
    path = os.path.join(os.path.dirname(_lib.__file__), "csrc", "build", "kernel_resources.json")
    if not os.path.exists(path):
        pytest.skip("library was not built in this tree")
    res = json.load(open(path))
    assert len(res) > 20
    for name, r in res.items():
        assert r.get("ScratchSize", 0) == 0, name
        assert r.get("VGPRs", 0) + r.get("AGPRs", 0) <= 512, name


def test_geometry_matches_reference_block_formats():
    L = _lib.lib()
    assert L.gq_abi_version() == 1
    for t, bpb, vpb in [(ggml.Q4_0, 18, 32), (ggml.Q8_0, 34, 32), (ggml.Q4_K, 144, 256), (ggml.Q6_K, 210, 256), (ggml.IQ4_NL, 18, 32)]:
        assert L.gq_bytes_per_block(t) == bpb == ggml.bytes_per_block(t)
        assert L.gq_values_per_block(t) == vpb == ggml.values_per_block(t)
    assert L.gq_row_bytes(ggml.Q8_0, 4096) == 4352
    assert L.gq_row_bytes(ggml.Q4_0, 4096) == 2304
    assert L.gq_row_bytes(ggml.Q4_K, 14336) == 8064
    assert L.gq_row_bytes(ggml.Q4_K, 4096) == 2304
    assert L.gq_row_bytes(ggml.Q4_K, 4128) == 0      # not a whole number of super-blocks
    assert L.gq_row_bytes(ggml.Q8_0, 0) == 0
    assert L.gq_row_bytes(99, 4096) == 0
    assert L.gq_bytes_per_block(99) == 0
    assert ggml.can_decompose(ggml.Q8_0) and ggml.can_decompose(ggml.Q4_0) and ggml.can_decompose(ggml.IQ4_NL)
    assert not ggml.can_decompose(ggml.Q4_K) and not ggml.can_decompose(ggml.Q6_K)   # ml/ggml/dequant.go:20-27


def check(*args):
    K = ctypes.c_int64(-1)
    rc = _lib.lib().gq_qdense_check(*args, ctypes.byref(K))
    return rc, K.value, _lib.lib().gq_last_error().decode()


def test_build_time_validation():
    # (type, x_dtype, M, x_last_dim, N, w_row_bytes, bias_len, act)
    assert check(ggml.Q8_0, _lib.F32, 1, 4096, 4096, 4352, -1, 0)[:2] == (_lib.OK, 4096)
    assert check(ggml.Q4_K, _lib.F32, 32, 14336, 4096, 8064, 4096, 3)[:2] == (_lib.OK, 14336)
    assert check(ggml.Q8_0, _lib.BF16, 2048, 4096, 4096, 4352, -1, 0)[:2] == (_lib.OK, 4096)
    assert check(ggml.Q4_0, _lib.F32, 0, 32, 2, 18, -1, 0)[0] == _lib.OK          # empty batch is fine
    # malformed -> hard error (the graph layer panics, core/graph/fused_ops.go:233-235)
    rc, _, msg = check(ggml.Q8_0, _lib.F32, 1, 4096, 4096, 4353, -1, 0)
    assert rc == _lib.ERR_INVALID and "whole number" in msg
    rc, _, msg = check(ggml.Q8_0, _lib.F32, 1, 4000, 4096, 4352, -1, 0)           # ml/ggml/dense.go:38-41
    assert rc == _lib.ERR_INVALID and "K=4096" in msg
    assert check(ggml.Q8_0, _lib.F32, 1, 4096, 4096, 4352, 4095, 0)[0] == _lib.ERR_INVALID
    assert check(ggml.Q8_0, _lib.F32, 1, 4096, 4096, 4352, -1, 6)[0] == _lib.ERR_INVALID
    assert check(ggml.Q8_0, _lib.F32, 1, 4096, 4096, 0, -1, 0)[0] == _lib.ERR_INVALID
    # valid but unsupported -> NotImplemented (caller falls back, core/graph/fused_ops.go:357-363)
    assert check(ggml.Q6_K, _lib.F32, 1, 256, 4, 210, -1, 0)[:2] == (_lib.OK, 256)
    assert check(13, _lib.F32, 1, 256, 4, 176, -1, 0)[0] == _lib.ERR_NOT_IMPLEMENTED   # Q5_K is not built
    assert check(ggml.Q8_0, 7, 1, 4096, 4096, 4352, -1, 0)[0] == _lib.ERR_NOT_IMPLEMENTED


def test_argument_errors_are_reported_before_any_device_work():
    L = _lib.lib()
    # bad K / type are diagnosed from the arguments alone, with or without a GPU
    assert L.gq_qdense_f32(ggml.Q8_0, 16, 1, 33, 16, 1, None, 0, 16, None) == _lib.ERR_INVALID
    assert b"multiple of the block size" in L.gq_last_error()
    assert L.gq_qdense_f32(99, 16, 1, 32, 16, 1, None, 0, 16, None) == _lib.ERR_NOT_IMPLEMENTED
    assert L.gq_qdense_bf16(ggml.Q4_K, 16, 1, 255, 16, 1, None, 0, 16, None) == _lib.ERR_INVALID
    assert L.gq_qdense_f32(ggml.Q8_0, 16, 1, 32, 16, 1, None, 9, 16, None) == _lib.ERR_INVALID
    assert L.gq_qdense_f32(ggml.Q8_0, None, 1, 32, 16, 1, None, 0, 16, None) == _lib.ERR_INVALID
    assert L.gq_qdense_f32(ggml.Q8_0, 16, 1, 32, 24, 1, None, 0, 16, None) == _lib.ERR_INVALID   # W not 16-B aligned
    assert L.gq_dequantize(ggml.Q4_0, 16, 2, 48, 16, None) == _lib.ERR_INVALID
    assert L.gq_dequantize(ggml.Q4_0, 16, -1, 32, 16, None) == _lib.ERR_INVALID
    assert L.gq_embedding_lookup(ggml.Q4_0, 16, 0, 32, 16, 3, 16, None, None) == _lib.ERR_INVALID
    assert L.gq_graph_begin(None) == _lib.ERR_INVALID
    assert L.gq_profile_end(None, None) == _lib.ERR_INVALID
    # empty problems succeed without touching a device
    assert L.gq_qdense_f32(ggml.Q8_0, None, 0, 32, None, 5, None, 0, None, None) == _lib.OK
    assert L.gq_dequantize(ggml.Q8_0, None, 0, 32, None, None) == _lib.OK


def test_argument_errors_of_the_calls_around_a_projection():
    L = _lib.lib()
    f = ctypes.c_float
    norm = _lib.RmsNormDesc(None, 1e-6, 0.0)
    bad_eps = _lib.RmsNormDesc(None, -1.0, 0.0)
    odd_gain = _lib.RmsNormDesc(18, 1e-6, 0.0)
    assert L.gq_rmsnorm_f32(16, 2, 0, None, f(1e-6), f(0), 16, None) == _lib.ERR_INVALID            # K = 0
    assert L.gq_rmsnorm_f32(16, 2, 8, None, f(-1.0), f(0), 16, None) == _lib.ERR_INVALID            # negative epsilon
    assert L.gq_rmsnorm_f32(None, 2, 8, None, f(1e-6), f(0), 16, None) == _lib.ERR_INVALID
    assert L.gq_rmsnorm_f32(None, 0, 8, None, f(1e-6), f(0), None, None) == _lib.OK                 # no rows
    # block dense: the checks of the dense call, then its own
    assert L.gq_qdense_block_f32(ggml.Q8_0, 16, 1, 33, ctypes.byref(norm), 16, 1, None, 0, None, 16, None) == _lib.ERR_INVALID
    assert L.gq_qdense_block_f32(99, 16, 1, 32, ctypes.byref(norm), 16, 1, None, 0, None, 16, None) == _lib.ERR_NOT_IMPLEMENTED
    assert L.gq_qdense_block_f32(ggml.Q8_0, 16, 1, 32, ctypes.byref(bad_eps), 16, 1, None, 0, None, 16, None) == _lib.ERR_INVALID
    assert b"epsilon" in L.gq_last_error()
    assert L.gq_qdense_block_f32(ggml.Q8_0, 16, 1, 32, ctypes.byref(odd_gain), 16, 1, None, 0, None, 16, None) == _lib.ERR_INVALID
    assert L.gq_qdense_block_f32(ggml.Q8_0, 16, 1, 32, None, 16, 1, None, 0, 18, 16, None) == _lib.ERR_INVALID   # residual alignment
    assert L.gq_qdense_block_f32(ggml.Q8_0, None, 0, 32, ctypes.byref(norm), None, 5, None, 0, None, None, None) == _lib.OK
    # gated: both matrices are checked
    assert L.gq_qdense_gated_f32(ggml.Q8_0, 16, 1, 32, None, 16, None, None, None, 1, 3, 16, None) == _lib.ERR_INVALID   # no up matrix
    assert L.gq_qdense_gated_f32(ggml.Q8_0, 16, 1, 32, None, 16, None, 24, None, 1, 3, 16, None) == _lib.ERR_INVALID     # up not aligned
    assert L.gq_qdense_gated_f32(ggml.Q8_0, 16, 1, 32, ctypes.byref(bad_eps), 16, None, 32, None, 1, 3, 16, None) == _lib.ERR_INVALID
    assert L.gq_qdense_gated_f32(13, 16, 1, 256, None, 16, None, 32, None, 1, 3, 16, None) == _lib.ERR_NOT_IMPLEMENTED
    assert L.gq_qdense_gated_f32(ggml.Q8_0, None, 0, 32, None, None, None, None, None, 5, 3, None, None) == _lib.OK
    # batched projections behind a norm
    d = (_lib.DenseDesc * 1)()
    d[0].type, d[0].act, d[0].dX, d[0].M, d[0].K, d[0].dW, d[0].N, d[0].dBias, d[0].dY = ggml.Q8_0, 0, 16, 1, 33, 16, 1, None, 16
    assert L.gq_qdense_norm_f32_batch(1, d, ctypes.byref(norm), None) == _lib.ERR_INVALID
    assert L.gq_qdense_norm_f32_batch(-1, None, ctypes.byref(norm), None) == _lib.ERR_INVALID
    assert L.gq_qdense_norm_f32_batch(0, None, ctypes.byref(norm), None) == _lib.OK
    d[0].K = 32
    assert L.gq_qdense_norm_f32_batch(1, d, ctypes.byref(bad_eps), None) == _lib.ERR_INVALID


def test_python_wrapper_maps_statuses_to_exceptions():
    with pytest.raises(_lib.HipqError) as e:
        _lib.check(_lib.lib().gq_qdense_f32(ggml.Q8_0, 16, 1, 33, 16, 1, None, 0, 16, None))
    assert e.value.status == _lib.ERR_INVALID and not isinstance(e.value, _lib.NotImplementedByBackend)
    with pytest.raises(_lib.NotImplementedByBackend):
        _lib.check(_lib.lib().gq_qdense_f32(99, 16, 1, 32, 16, 1, None, 0, 16, None))


def test_activation_mapping_quirks():
    from gomlx_amd.nn import Activation
    # activation.Type.ToBackend, ml/layers/activation/activation.go:58-75
    assert Activation.GELU.to_backend() == Activation.GELU_APPROX.to_backend() == 1
    assert Activation.SWISH.to_backend() == Activation.SILU.to_backend() == 3
    assert Activation.RELU.to_backend() == 2 and Activation.HARD_SWISH.to_backend() == 4 and Activation.TANH.to_backend() == 5
    for dropped in (Activation.SIGMOID, Activation.HARD_SIGMOID, Activation.LEAKY_RELU, Activation.SELU, Activation.SWIGLU):
        assert dropped.to_backend() == 0
