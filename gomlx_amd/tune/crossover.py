"""Times one dense entry point over a list of batch sizes on one (type, K, N), weights rotating over copies.

    python -m gomlx_amd.tune.crossover Q4_K 4096 4096 f32 64,96,128,160,192,256
    python -m gomlx_amd.tune.crossover Q4_K 4096 14336 gated 64,96,128,160,192,256      # act(x.Wgate) * (x.Wup), fp32 activations

Run it under the tuning knobs (GOMLX_HIPQ_SPLIT_K_TO, GOMLX_HIPQ_GATED_TWO_PASS_FROM, GOMLX_HIPQ_TWO_PASS_MIN_ROWS, GOMLX_HIPQ_GEMM_TILE)
to compare routes;
the tables of measured crossovers in csrc/api.hip and csrc/gemm_dma.hip come from runs of this kind."""
import ctypes
import os
import sys

import torch

from gomlx_amd import _lib, ggml, synth


def main(argv):
    tname, K, N, bf16, gated = argv[0], int(argv[1]), int(argv[2]), argv[3] == "bf16", argv[3] == "gated"
    Ms = [int(v) for v in argv[4].split(",")]
    if os.environ.get("GOMLX_HIPQ_LIBRARY"):
        # another build of the library (an A/B of two builds on one machine), possibly an older one that lacks newer
        # entry points: only what this tool calls is bound
        L = ctypes.CDLL(os.path.abspath(os.environ["GOMLX_HIPQ_LIBRARY"]))
        for name, restype, argtypes in _lib.SIGNATURES:
            if hasattr(L, name):
                getattr(L, name).restype, getattr(L, name).argtypes = restype, argtypes
        _lib._lib = L
    else:
        L = _lib.lib()
    _lib.init(0)
    t = getattr(ggml, tname)
    W0 = torch.from_numpy(synth.weights(t, 1, N, K)).cuda()
    Ws = [W0.clone() for _ in range(min(max(2, (600 << 20) // W0.numel()), 24))]
    st = torch.cuda.Stream()
    dense = L.gq_qdense_bf16 if bf16 else L.gq_qdense_f32

    def fn(t, xp, M, K, Wp, N, bias, act, yp, stream):
        if not gated:
            return dense(t, xp, M, K, Wp, N, bias, act, yp, stream)
        return L.gq_qdense_gated_f32(t, xp, M, K, None, Wp, None, Wup.data_ptr(), None, N, 3, yp, stream)

    Wup = W0.clone()
    out = []
    for M in [Ms[0]] + Ms:  # (the first pass over the first size warms the process up and is dropped)
        x = torch.randn(M, K, device="cuda")
        if bf16:
            x = x.to(torch.bfloat16)
        y = torch.empty(M, N, device="cuda")
        with torch.cuda.stream(st):
            for i in range(3):  # (creates the stream's workspace before anything is recorded)
                _lib.check(fn(t, x.data_ptr(), M, K, Ws[i % len(Ws)].data_ptr(), N, None, 0, y.data_ptr(), st.cuda_stream))
            torch.cuda.synchronize()
            # 20 dependent calls recorded once and replayed: what a compiled graph's Execute costs, without the host's launch time
            _lib.check(L.gq_graph_begin(st.cuda_stream))
            for i in range(20):
                _lib.check(fn(t, x.data_ptr(), M, K, Ws[i % len(Ws)].data_ptr(), N, None, 0, y.data_ptr(), st.cuda_stream))
            graph = ctypes.c_void_p()
            _lib.check(L.gq_graph_end(st.cuda_stream, ctypes.byref(graph)))
            _lib.check(L.gq_graph_launch(graph, st.cuda_stream))
            torch.cuda.synchronize()
            best = None
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(st)
                _lib.check(L.gq_graph_launch(graph, st.cuda_stream))
                e1.record(st)
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) * 1e3 / 20
                best = us if best is None else min(best, us)
            _lib.check(L.gq_graph_destroy(graph))
        out.append(f"{M}:{best:.1f}")
    knobs = {k: v for k, v in os.environ.items() if k.startswith("GOMLX_HIPQ_")}
    print(tname, K, N, argv[3], knobs, " ".join(out[1:]), flush=True)


if __name__ == "__main__":
    main(sys.argv[1:])
