#!/usr/bin/env python3
"""Benchmark of the quantized Dense hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1] [--others]

--config takes c0 .. c4 (the BASELINE.json configurations), prefill (C3's shape with fp32 activations), ffn (the gated feed-forward front of
a decoder layer: the callers around the two projections folded into one launch) or layer (the
seven projections of C4 in the order and with the dependencies of a decoder layer).

A "step" is one quantized Dense call (one pass over one weight matrix) on synthetic data that
is already resident in HBM.  The headline workload is BASELINE.json configs[1]: Q4_0 decode
GEMV, batch 1, K=4096 -> N=14336.  Steps rotate over enough distinct weight copies (> 512 MB)
that every pass streams its weights from HBM rather than from the 256 MB Infinity Cache.

Prints ONE JSON line.  `value` is weight-GB/s over the wall clock of the K timed steps
(submitted as one recorded HIP graph unless --no-graph).  `roofline` is the dominant kernel's
own rate: algorithmic weight bytes per launch / mean kernel duration from start/stop HIP
events attached to each launch on its stream (a second pass over the same K steps).
The kernel time is taken two ways with HIP events and the smaller is used (both are upper
bounds): events bracketing every launch, and two events around the timed region divided by K.
`cpu_baseline` times the CPU oracle's fused fp32 restatement on the host cores (rank 0, N=1).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0

# HBM-side traffic per step in bytes, from hardware counters: two `rocprofv3 --pmc` passes per
# workload (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch, summed over the step's kernels), each
# scaled by what the same counter reads for the 64 MiB copy of --copy-calibration (FETCH_SIZE
# reads 32780.5 KiB for 65536 KiB copied: factor 1.99924; WRITE_SIZE reads 65536.0: factor 1.0).
# The readings are summarised under profiles/; they are properties of the kernels' access
# pattern, not of a particular run, and are re-measured whenever a kernel changes.
_KIB, _FETCH_SCALE, _WRITE_SCALE = 1024, 65536.0 / 32780.5, 1.0
COUNTER_KIB = {  # workload -> (FETCH_SIZE, WRITE_SIZE) raw counter KiB per step
    "c0": (8811.9, 16.0),
    "c1": (16262.6, 56.0),
    "c2": (19876.6 + 1869.1 + 921.1, 3584.0 + 512.0 + 925.8),
    "c3": (74726.7, 32768.0),
    "c4": (60543.5, 168.0),
    "prefill": (4628.9 + 16401.2 + 82465.3, 32768.0 + 16448.0 + 32768.0),
    "ffn": (32484.0, 56.0),
    "layer": (7126.2 + 4756.1 + 32483.6 + 16449.7, 24.0 + 16.0 + 56.0 + 16.0),
}


def measured_traffic(name):
    if name not in COUNTER_KIB:
        return None
    f, w = COUNTER_KIB[name]
    return int(round((f * _FETCH_SCALE + w * _WRITE_SCALE) * _KIB))


# name -> (ggml type name, M, K, N, activation dtype, bound)
CONFIGS = {
    "c0": ("Q8_0", 1, 4096, 4096, "f32", "hbm"),
    "c1": ("Q4_0", 1, 4096, 14336, "f32", "hbm"),
    "c2": ("Q4_K", 32, 14336, 4096, "f32", "hbm"),
    "c3": ("Q8_0", 2048, 4096, 4096, "bf16", "mfma"),
    "prefill": ("Q4_K", 2048, 4096, 4096, "f32", "mfma"),
}
C4_SHAPES = [(4096, 4096), (4096, 1024), (4096, 1024), (4096, 4096), (4096, 14336), (4096, 14336), (14336, 4096)]
WORKLOAD_TEXT = {
    "c0": "configs[0]: Q8_0 dense GEMV, x f32 [1,4096], W [4096,4096]",
    "c1": "configs[1]: Q4_0 dense GEMV, batch 1, K=4096 -> N=14336",
    "c2": "configs[2]: Q4_K dense, decode batch M=32, K=14336 -> N=4096",
    "c3": "configs[3]: Q8_0 prefill GEMM, M=2048 bf16, K=4096, N=4096",
    "c4": "configs[4]: seven Q4_K projections of a Llama-3-8B layer, batch 1",
    "prefill": "C3's shape with fp32 activations and Q4_K weights (M=2048, K=4096, N=4096): weights to an fp16 image, activations "
               "to scaled fp16 rows, fp16 MFMA GEMM (three launches)",
    "layer": "the seven Q4_K projections of a Llama-3-8B layer as a decoder runs them, batch 1: four dependent launches "
             "(RMSNorm + q/k/v, o + residual, RMSNorm + gate/up + SiLU*mul, down + residual)",
    "ffn": "gated feed-forward front of a Llama-3-8B layer, batch 1: RMSNorm, Q4_K gate and up 4096 -> 14336, SiLU(gate) * up, one launch",
}


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--config", default="c1", choices=sorted(list(CONFIGS) + ["c4", "ffn", "layer"]))
    p.add_argument("--rows", type=int, default=1, help="activation rows of the ffn and layer workloads (a decode batch); default 1")
    p.add_argument("--others", action="store_true", help="also measure the other configurations (reported under 'others')")
    p.add_argument("--no-graph", action="store_true", help="submit the timed steps one call at a time")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    p.add_argument("--hot", action="store_true", help="single weight buffer (Infinity-Cache resident) instead of the cold rotation")
    p.add_argument("--copy-calibration", action="store_true",
                   help="instead of the benchmark, run a plain 64 MiB device-to-device copy kernel --steps times: the known-size "
                        "workload that hardware counter readings (FETCH_SIZE / WRITE_SIZE) are scaled by")
    return p.parse_args()


class Problem:
    """One (x, W-rotation, y) set resident on the GPU plus the launch closure."""

    def __init__(self, torch, name, hot=False, rows=1):
        from gomlx_amd import _lib, ggml, synth
        import numpy as np
        self.torch, self.name = torch, name
        self.L = _lib.lib()
        self.check = _lib.check
        self.rows = rows if name in ("ffn", "layer") else 1
        if name in ("c4", "layer"):
            shapes = [("Q4_K", self.rows, K, N) for K, N in C4_SHAPES]
            self.dtype, self.bound = "f32", "hbm"
            self.gain = torch.ones(4096, device="cuda")
        elif name == "ffn":  # gate and up matrices of one feed-forward block
            shapes = [("Q4_K", self.rows, 4096, 14336)] * 2
            self.dtype, self.bound = "f32", "hbm"
            self.gain = torch.from_numpy((synth.normal(1200, 0, 4096) * 0.5 + 1.0).astype(np.float32)).cuda()
        else:
            tn, M, K, N, self.dtype, self.bound = CONFIGS[name]
            shapes = [(tn, M, K, N)]
        self.parts = []
        seed = 1000 + (int(name[1]) if name[0] == "c" else {"layer": 4, "ffn": 5, "prefill": 6}[name])
        total_w = 0
        for i, (tn, M, K, N) in enumerate(shapes):
            t = getattr(ggml, tn)
            W = torch.from_numpy(synth.weights(t, seed + i, N, K)).cuda()
            x = torch.from_numpy(synth.activations(seed + 100 + i, M, K)).cuda()
            if self.dtype == "bf16":
                x = x.to(torch.bfloat16)
            y = torch.empty((M, N), dtype=torch.float32, device="cuda")
            self.parts.append(dict(t=t, M=M, K=K, N=N, W=[W], x=x, y=y, wbytes=W.numel()))
            total_w += W.numel()
        self.weight_bytes = total_w
        self.flops = sum(2 * p["M"] * p["K"] * p["N"] for p in self.parts)
        # cold rotation: distinct copies (rows rolled) until the set exceeds 2 x Infinity Cache
        self.copies = 1 if hot else max(2, -(-(512 << 20) // total_w) + 1)
        for p in self.parts:
            for c in range(1, self.copies):
                p["W"].append(torch.roll(p["W"][0], shifts=c, dims=0).contiguous())
        # one explicit stream for everything: warm-up, the recorded graph and the timed launches
        # (per-stream workspaces of the library must exist before a recording starts)
        self.tstream = torch.cuda.Stream()
        self.stream = self.tstream.cuda_stream
        torch.cuda.synchronize()

    def launch(self, step):
        c = step % self.copies
        if self.name == "c4":  # the seven independent projections go out as one batched submission
            from gomlx_amd import _lib
            descs = (_lib.DenseDesc * len(self.parts))()
            for d, p in zip(descs, self.parts):
                d.type, d.act, d.dX, d.M, d.K = p["t"], 0, p["x"].data_ptr(), p["M"], p["K"]
                d.dW, d.N, d.dBias, d.dY = p["W"][c].data_ptr(), p["N"], None, p["y"].data_ptr()
            self.check(self.L.gq_qdense_f32_batch(len(self.parts), descs, self.stream))
            return
        if self.name == "layer":
            # q, k, v, o, gate, up, down in C4's order; the attention between v and o is not part of this path: o reads a
            # fixed vector of the right shape.  Outputs feed the next call where the shapes chain (o -> gate/up -> down).
            from gomlx_amd import _lib
            q, k, v, o, g, u, d = self.parts
            norm = _lib.RmsNormDesc(self.gain.data_ptr(), 1e-5, 0.0)
            descs = (_lib.DenseDesc * 3)()
            for ds, p in zip(descs, (q, k, v)):
                ds.type, ds.act, ds.dX, ds.M, ds.K = p["t"], 0, q["x"].data_ptr(), self.rows, p["K"]
                ds.dW, ds.N, ds.dBias, ds.dY = p["W"][c].data_ptr(), p["N"], None, p["y"].data_ptr()
            self.check(self.L.gq_qdense_norm_f32_batch(3, descs, ctypes.byref(norm), self.stream))
            self.check(self.L.gq_qdense_block_f32(o["t"], o["x"].data_ptr(), self.rows, o["K"], None, o["W"][c].data_ptr(), o["N"], None, 0,
                                                  q["x"].data_ptr(), o["y"].data_ptr(), self.stream))
            self.check(self.L.gq_qdense_gated_f32(g["t"], o["y"].data_ptr(), self.rows, g["K"], ctypes.byref(norm), g["W"][c].data_ptr(), None,
                                                  u["W"][c].data_ptr(), None, g["N"], 3, g["y"].data_ptr(), self.stream))
            self.check(self.L.gq_qdense_block_f32(d["t"], g["y"].data_ptr(), self.rows, d["K"], None, d["W"][c].data_ptr(), d["N"], None, 0,
                                                  o["y"].data_ptr(), d["y"].data_ptr(), self.stream))
            return
        if self.name == "ffn":
            from gomlx_amd import _lib
            g, u = self.parts
            norm = _lib.RmsNormDesc(self.gain.data_ptr(), 1e-5, 0.0)
            self.check(self.L.gq_qdense_gated_f32(g["t"], g["x"].data_ptr(), self.rows, g["K"], ctypes.byref(norm), g["W"][c].data_ptr(), None,
                                                  u["W"][c].data_ptr(), None, g["N"], 3, g["y"].data_ptr(), self.stream))
            return
        for p in self.parts:
            fn = self.L.gq_qdense_bf16 if self.dtype == "bf16" else self.L.gq_qdense_f32
            self.check(fn(p["t"], p["x"].data_ptr(), p["M"], p["K"], p["W"][c].data_ptr(), p["N"], None, 0,
                          p["y"].data_ptr(), self.stream))

    def run(self, steps, warmup, use_graph):
        torch, L = self.torch, self.L
        for s in range(warmup):
            self.launch(s)
        torch.cuda.synchronize()
        graph = None
        if use_graph:
            if warmup == 0:
                self.launch(0)  # creates the stream's workspace, if the path needs one
                torch.cuda.synchronize()
            self.check(L.gq_graph_begin(self.stream))
            for s in range(steps):
                self.launch(warmup + s)
            g = ctypes.c_void_p()
            self.check(L.gq_graph_end(self.stream, ctypes.byref(g)))
            graph = g
            if warmup > 0:  # untimed first replay: uploads the graph
                self.check(L.gq_graph_launch(graph, self.stream))
            torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record(self.tstream)  # events on the stream the kernels are launched on
        if graph is not None:
            self.check(L.gq_graph_launch(graph, self.stream))
        else:
            for s in range(steps):
                self.launch(warmup + s)
        ev1.record(self.tstream)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        self.region_us_per_step = ev0.elapsed_time(ev1) * 1e3 / steps
        if graph is not None:
            self.check(L.gq_graph_destroy(graph))
        # second pass over the same steps: per-launch start/stop events on the launch stream
        self.check(L.gq_profile_begin())
        for s in range(steps):
            self.launch(warmup + s)
        n, us = ctypes.c_int(0), ctypes.c_double(0.0)
        self.check(L.gq_profile_end(ctypes.byref(n), ctypes.byref(us)))
        self.bracketed_us_per_step = us.value / steps
        # Both figures bound the mean kernel time from above: the bracketed one carries the cost of
        # the two event packets around every launch, the region one the gaps between launches.
        kernel_us_per_step = min(self.bracketed_us_per_step, self.region_us_per_step)
        return wall, kernel_us_per_step, n.value // steps

    def report(self, wall, kernel_us, steps):
        out = {}
        if self.bound == "hbm":
            out["metric"], out["unit"] = "dense GEMV weight-GB/s", "GB/s"
            out["value"] = self.weight_bytes * steps / wall / 1e9
            ach = self.weight_bytes / (kernel_us * 1e-6) / 1e9
            out["roofline"] = {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                               "frac": ach / HBM_PEAK_GBS, "traffic": measured_traffic(self.name) if self.rows == 1 else None,
                               "algorithmic_bytes_per_launch": self.weight_bytes, "kernel_us": kernel_us}
        else:
            out["metric"], out["unit"] = "prefill GEMM TFLOP/s", "TFLOP/s"
            out["value"] = self.flops * steps / wall / 1e12
            ach = self.flops / (kernel_us * 1e-6) / 1e12
            out["roofline"] = {"bound": "mfma", "achieved": ach, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                               "frac": ach / MFMA_BF16_PEAK_TFLOPS, "traffic": measured_traffic(self.name),
                               "algorithmic_flops_per_launch": self.flops, "kernel_us": kernel_us}
        out["roofline"]["kernel_us_bracketed"] = self.bracketed_us_per_step
        out["roofline"]["kernel_us_region"] = self.region_us_per_step
        out["ms_per_step"] = wall / steps * 1e3
        return out


def cpu_baseline(name):
    """The CPU oracle's fused fp32 restatement on the host cores (checker code used as a
    reported baseline only): >= 2 warm-ups, then >= 5 runs and >= 3 s, like the reference's own
    timing protocol (internal/perf/dotgeneral_perf_test.go:366-381), capped at ~25 s."""
    import numpy as np
    from gomlx_amd import ggml, synth
    from oracle import ggml_oracle as oracle
    cores = min(os.cpu_count() or 1, 16)
    if name in ("c4", "layer"):
        shapes = [("Q4_K", 1, K, N) for K, N in C4_SHAPES]
    elif name == "ffn":  # the two projections; the normalisation and the product are negligible beside them
        shapes = [("Q4_K", 1, 4096, 14336)] * 2
    else:
        tn, M, K, N, _, _ = CONFIGS[name]
        shapes = [(tn, M, K, N)]
    sample = "full workload"
    if name in ("c3", "prefill"):  # 34 GMAC per pass is minutes of CPU time: a 64-row slice of the 2048 activations
        shapes = [(CONFIGS[name][0], 64, 4096, 4096)]
        sample = "64 of the 2048 activation rows (1/32 of the FLOPs), all of W"
    probs = []
    for i, (tn, M, K, N) in enumerate(shapes):
        t = getattr(ggml, tn)
        probs.append((t, synth.activations(5 + i, M, K), synth.weights(t, 6 + i, N, K)))
    wbytes = sum(p[2].size for p in probs)
    flops = sum(2 * p[1].shape[0] * p[1].shape[1] * p[2].shape[0] for p in probs)

    def once():
        for t, x, W in probs:
            oracle.c_qdense(t, x, W, None, 0, f32acc_threads=cores)

    once(); once()
    runs, t0 = 0, time.perf_counter()
    while True:
        once()
        runs += 1
        el = time.perf_counter() - t0
        if (runs >= 5 and el >= 3.0) or el >= 25.0:
            break
    per = el / runs
    if name in ("c3", "prefill"):
        return {"value": flops / per / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
                "sample": f"{sample}; {runs} runs, {per * 1e3:.2f} ms each"}
    return {"value": wbytes / per / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"{sample}; {runs} runs, {per * 1e3:.2f} ms each"}


def copy_calibration(torch, steps):
    """A copy kernel of known size: each launch reads 64 MiB and writes 64 MiB (an elementwise
    `dst = src + 0` over 16 Mi floats; sources rotate over 10 buffers so reads come from HBM)."""
    n = (64 << 20) // 4
    srcs = [torch.full((n,), float(i), device="cuda") for i in range(10)]
    dst = torch.empty(n, device="cuda")
    torch.cuda.synchronize()
    for s in range(steps):
        torch.add(srcs[s % len(srcs)], 0.0, out=dst)
    torch.cuda.synchronize()
    print(json.dumps({"copy_calibration": True, "launches": steps, "read_bytes_per_launch": n * 4, "write_bytes_per_launch": n * 4}))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path is a single-GPU kernel: rows of W are independent, so it "
              "would shard by output features); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; there is no CPU fallback for the product path", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    if args.copy_calibration:
        copy_calibration(torch, args.steps)
        return
    from gomlx_amd import _lib
    _lib.init(0)

    def measure(name):
        prob = Problem(torch, name, hot=args.hot, rows=args.rows)
        wall, kus, launches = prob.run(args.steps, args.warmup, not args.no_graph)
        rep = prob.report(wall, kus, args.steps)
        rep["weight_copies"] = prob.copies
        rep["launches_per_step"] = launches
        del prob
        torch.cuda.empty_cache()
        return rep

    rep = measure(args.config)
    tn = "Q4_K" if args.config in ("c4", "ffn", "layer") else CONFIGS[args.config][0]
    line = {
        "metric": rep["metric"], "value": rep["value"], "unit": rep["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": rep["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"c3": "bf16", "prefill": "f16"}.get(args.config, "f32"), "data": "synthetic",
        "config": {"workload": WORKLOAD_TEXT[args.config] + (f" [run with {args.rows} activation rows]" if args.rows != 1 and args.config in ("ffn", "layer") else ""),
                   "ggml_type": tn,
                   "weights": "cache-resident single buffer" if args.hot else
                   f"cold: rotation over {rep['weight_copies']} distinct weight copies",
                   "submission": "eager" if args.no_graph else "one recorded HIP graph of all timed steps",
                   "launches_per_step": rep["launches_per_step"]},
        "roofline": rep["roofline"],
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(args.config)
    if args.others:
        others = {}
        for name in ["c0", "c1", "c2", "c3", "c4", "prefill", "ffn", "layer"]:
            if name == args.config:
                continue
            steps = args.steps if name not in ("c3", "prefill") else max(10, args.steps // 10)
            saved = args.steps
            args.steps = steps
            r = measure(name)
            args.steps = saved
            others[name] = {"workload": WORKLOAD_TEXT[name], "metric": r["metric"], "value": r["value"], "unit": r["unit"],
                            "ms_per_step": r["ms_per_step"], "roofline": r["roofline"], "steps": steps}
        line["others"] = others
    print(json.dumps(line))


if __name__ == "__main__":
    main()
