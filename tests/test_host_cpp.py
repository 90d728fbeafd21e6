"""Runs the C++ host layer's own test program (gomlx_amd/host/hipq_backend_test.cpp), which
mirrors the reference's Go tests of nn.QuantizedDense / nn.QuantizedGather
(ml/nn/quantized_dense_test.go:272-452, ml/nn/quantized_gather_test.go:17-169) above the C ABI."""
import os
import subprocess

import pytest

from gomlx_amd import build


def _binary():
    if not os.path.exists(build.HOST_TEST):
        if not os.path.exists(build.LIB):
            build.build(verbose=False)
        else:
            build.build_host_test(verbose=False)
    return build.HOST_TEST


def _run(*args, binary=None):
    r = subprocess.run([binary or _binary(), *args], capture_output=True, text=True, timeout=100)
    print(r.stdout)
    print(r.stderr)
    return r


def test_host_layer_build_time_rules():
    """Graph-build validation, ErrNotImplemented vs hard errors, GOMLX_FUSION: no GPU needed."""
    r = _run("--build-only")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "0 failed" in r.stdout and "FAIL" not in r.stdout


def test_workspace_bookkeeping():
    """Scratch-memory pool against fake device hooks: growth, graph pinning, stream destruction, and two host threads
    on one stream never interleaving their launch sequences."""
    _binary()
    if not os.path.exists(build.WORKSPACE_TEST):
        build.build_host_test(verbose=False)
    r = _run(binary=build.WORKSPACE_TEST)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "0 failed" in r.stdout and "FAIL" not in r.stdout


def _sanitized(name):
    path = build.sanitized_path(name)
    if not os.path.exists(path):
        if not os.path.exists(build.LIB):
            build.build(verbose=False)
        else:
            build.build_sanitized(verbose=False)
    return path


def _clean(r):
    assert r.returncode == 0, r.stdout + r.stderr
    assert "0 failed" in r.stdout and "FAIL" not in r.stdout
    for word in ("ThreadSanitizer", "AddressSanitizer", "LeakSanitizer", "runtime error"):
        assert word not in r.stderr, r.stderr


def test_workspace_bookkeeping_under_thread_sanitizer():
    """Two host threads on one stream, recordings, growth and destruction with every access to the pool's shared state
    watched for data races (the executor may compile and run from many goroutines, core/graph/exec.go:121-125)."""
    _clean(_run(binary=_sanitized("workspace_test_tsan")))


def test_workspace_bookkeeping_under_address_sanitizer():
    _clean(_run(binary=_sanitized("workspace_test_asan")))


def test_host_layer_build_time_rules_under_address_sanitizer():
    """The C++ host layer's graph-build validation and fallback rules with address and undefined-behaviour checks on."""
    _clean(_run("--build-only", binary=_sanitized("hipq_backend_test_asan")))


def test_oracle_under_address_sanitizer():
    """The oracle's C code on exactly-sized buffers with random bytes in every packed field (oracle/oracle_selftest.c)."""
    odir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")
    r = subprocess.run(["make", "-C", odir, "oracle_selftest_asan"], capture_output=True, text=True, timeout=200)
    assert r.returncode == 0, r.stdout + r.stderr
    _clean(_run(binary=os.path.join(odir, "oracle_selftest_asan")))


@pytest.mark.gpu
def test_host_layer_reference_cases_on_gpu():
    r = _run()
    assert r.returncode == 0, r.stdout + r.stderr
    assert "0 failed" in r.stdout and "FAIL" not in r.stdout
    assert "QuantizedDense_GGML_IQ4NL/basic" in r.stdout and "LayerGraph/independent_and_chained" in r.stdout
