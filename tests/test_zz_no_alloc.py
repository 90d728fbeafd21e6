"""The entry point that allocates nothing (gq_qdense_f32_static) against gq_qdense_f32, through the C ABI.

Same kernels, so the results must be bit-identical; the scratch memory is the library's fixed device
array, which keeps the previous call's contents: two calls in a row, the second smaller, both checked.
Collected last on purpose (a failure here must not hide the tests before it)."""
import numpy as np
import pytest

from gomlx_amd import _lib, ggml, synth

pytestmark = pytest.mark.gpu


def _dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _both(torch, oracle, t, M, K, N, seed, act=0, with_bias=True):
    L = _lib.lib()
    W, x = synth.weights(t, seed, N, K), synth.activations(seed + 1, M, K)
    bias = synth.normal(seed + 2, 0, N).astype(np.float32) * 0.1 if with_bias else None
    Wd, xd = _dev(torch, W), _dev(torch, x)
    bd = _dev(torch, bias) if with_bias else None
    y_ref = torch.full((M, N), float("nan"), device="cuda")
    y_sta = torch.full((M, N), float("nan"), device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    bp = bd.data_ptr() if with_bias else None
    _lib.check(L.gq_qdense_f32(t, xd.data_ptr(), M, K, Wd.data_ptr(), N, bp, act, y_ref.data_ptr(), stream))
    _lib.check(L.gq_qdense_f32_static(t, xd.data_ptr(), M, K, Wd.data_ptr(), N, bp, act, y_sta.data_ptr(), stream))
    torch.cuda.synchronize()
    a, b = y_ref.cpu().numpy(), y_sta.cpu().numpy()
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (ggml.name(t), M, K, N)
    want = oracle.c_qdense(t, x, W, bias, act)
    pre = oracle.c_qdense(t, x, W, bias, 0)
    scale = max(float(np.max(np.abs(want))), float(np.max(np.abs(pre))))
    assert float(np.max(np.abs(b.astype(np.float64) - want))) / scale < 1e-3


def test_static_scratch_entry_matches_the_allocating_one(gpu, oracle):
    """Split-K batches (the path with scratch memory): a larger call, then a smaller one on the same array."""
    for t in (ggml.Q4_K, ggml.Q8_0, ggml.Q4_0, ggml.Q6_K, ggml.IQ4_NL):
        _both(gpu, oracle, t, 32, 4096, 1024, 9100 + t, act=3)
        _both(gpu, oracle, t, 9, 2048, 512, 9200 + t, act=0, with_bias=False)
    # decode rows take no scratch at all and pass through unchanged
    _both(gpu, oracle, ggml.Q4_K, 1, 4096, 512, 9300)


def _ws_stats(L):
    import ctypes
    live, streams = ctypes.c_size_t(0), ctypes.c_int(0)
    _lib.check(L.gq_workspace_stats(ctypes.byref(live), ctypes.byref(streams)))
    return live.value, streams.value


def test_static_scratch_entry_allocates_nothing(gpu, oracle):
    """The property the entry point exists for.  On a stream the library has never seen (no workspace exists for it, so a
    call that fell through to the per-stream pool would have to create one), split-K calls go through the static entry
    first: the pool's books (bytes held, streams known) and the device's free memory must not move, and the results must
    be right.  The first call loads the kernels' code (the runtime may take device memory for that), so free memory is
    compared across the second, larger call."""
    import ctypes
    torch = gpu
    L = _lib.lib()
    sp = ctypes.c_void_p()
    _lib.check(L.gq_stream_create(ctypes.byref(sp)))
    try:
        t = ggml.Q4_K
        cases = []
        for M, K, N, seed in ((9, 2048, 512, 9400), (32, 4096, 2048, 9410)):
            W, x = synth.weights(t, seed, N, K), synth.activations(seed + 1, M, K)
            cases.append((M, K, N, x, W, _dev(torch, x), _dev(torch, W), torch.full((M, N), float("nan"), device="cuda")))
        torch.cuda.synchronize()
        books = _ws_stats(L)
        free_before = None
        for i, (M, K, N, x, W, xd, Wd, y) in enumerate(cases):
            if i == 1:
                free_before = torch.cuda.mem_get_info()[0]
            _lib.check(L.gq_qdense_f32_static(t, xd.data_ptr(), M, K, Wd.data_ptr(), N, None, 0, y.data_ptr(), sp))
            _lib.check(L.gq_sync(sp))
            assert _ws_stats(L) == books, "the static entry point touched the workspace pool"
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated during the call"
        for M, K, N, x, W, xd, Wd, y in cases:
            want = oracle.c_qdense(t, x, W)
            assert float(np.max(np.abs(y.cpu().numpy().astype(np.float64) - want))) / float(np.max(np.abs(want))) < 1e-3
        # the allocating entry point on the same stream does create a workspace: the books do see what they are meant to see
        M, K, N, x, W, xd, Wd, y = cases[1]
        y2 = torch.full((M, N), float("nan"), device="cuda")
        _lib.check(L.gq_qdense_f32(t, xd.data_ptr(), M, K, Wd.data_ptr(), N, None, 0, y2.data_ptr(), sp))
        _lib.check(L.gq_sync(sp))
        after = _ws_stats(L)
        assert after[0] > books[0] and after[1] == books[1] + 1
        assert torch.equal(y, y2)
    finally:
        _lib.check(L.gq_stream_destroy(sp))


def test_static_scratch_entry_rejects_what_does_not_fit(gpu):
    L = _lib.lib()
    t, M, K, N = ggml.Q8_0, 512, 4096, 4096  # two-pass GEMM: a 32 MiB weight image
    W = gpu.zeros((N, ggml.row_bytes(t, K)), dtype=gpu.uint8, device="cuda")
    x = gpu.zeros((M, K), device="cuda")
    y = gpu.full((M, N), 7.0, device="cuda")
    rc = L.gq_qdense_f32_static(t, x.data_ptr(), M, K, W.data_ptr(), N, None, 0, y.data_ptr(), gpu.cuda.current_stream().cuda_stream)
    assert rc == _lib.ERR_INVALID
    assert b"static buffer" in L.gq_last_error()
    gpu.cuda.synchronize()
    assert float(y.min()) == 7.0 and float(y.max()) == 7.0  # nothing was launched
