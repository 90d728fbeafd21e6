#!/usr/bin/env python3
"""Benchmark of the quantized Dense hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c4] [--no-others] [--all]

Workloads: c0 .. c4 are the BASELINE.json configurations; prefill is C3's shape with fp32
activations and Q4_K weights; ffn is the gated feed-forward front of a decoder layer in one
launch; layer is C4's seven projections in the order and with the dependencies of a decoder layer.

The headline (--config, default c4) is the largest decode GEMV configuration in a format the
metric names: the seven Q4_K projections of a Llama-3-8B layer at batch 1, 122.7 MB of weights in
one batched submission.  The other BASELINE configurations (c0 .. c3) are measured in the same run
and reported under "others" (--no-others skips them, --all adds prefill / ffn / layer).

A "step" is one pass of the workload over synthetic data that is already resident in HBM.  Steps
rotate over enough distinct weight copies (> 512 MB) that every pass streams its weights from HBM
rather than from the 256 MB Infinity Cache.

Prints ONE JSON line.  `value` is weight-GB/s (or TFLOP/s) over the wall clock of exactly K timed
steps, submitted as one recorded HIP graph unless --no-graph.  `roofline` is the dominant kernels'
own rate: algorithmic weight bytes (or FLOP) per step / kernel time per step, the latter measured
live with HIP events on the launch stream, two ways, the smaller taken (both bound it from above):
start/stop events attached to every launch, and two events around a replay of the K steps.
Per workload the line also carries: the same measurement with a single weight buffer, labelled
cache-resident (NOT the metric); the time a plain read-only kernel takes for the same bytes (the
rate this chip hands a one-shot kernel of that size, gomlx_amd/csrc/yardstick.hip); the HBM-side
traffic from hardware counters (read from profiles/traffic.json, where the profiling runs put it);
shader / memory clocks and socket power sampled while the workload loops.
`cpu_baseline` times the CPU oracle's fused fp32 restatement (kind "port": the reference is Go and
no Go toolchain exists here) on the host cores, on the same seeded inputs as the GPU leg.
"""
from __future__ import annotations

import argparse
import ctypes
import glob
import json
import os
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0

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
    "c4": "configs[4]: seven Q4_K projections of a Llama-3-8B layer, batch 1 (q, k, v, o, gate, up, down: 122.7 MB of weights, one batched submission)",
    "prefill": "C3's shape with fp32 activations and Q4_K weights (M=2048, K=4096, N=4096): weights to an fp16 image, activations "
               "to scaled fp16 rows, fp16 MFMA GEMM (three launches)",
    "layer": "the seven Q4_K projections of a Llama-3-8B layer as a decoder runs them, batch 1: four dependent launches "
             "(RMSNorm + q/k/v, o + residual, RMSNorm + gate/up + SiLU*mul, down + residual)",
    "ffn": "gated feed-forward front of a Llama-3-8B layer, batch 1: RMSNorm, Q4_K gate and up 4096 -> 14336, SiLU(gate) * up, one launch",
}
# What the path computes in (inputs and outputs are fp32 unless stated): this is `dtype` of the JSON line.
ARITHMETIC = {
    "c0": "f32 in/out; x -> 16-bit block fixed point (two int8 limbs per 32 values), v_dot4_i32_i8 against the int8 codes, i32 sums scaled and added in f32",
    "c1": "f32 in/out; x -> 16-bit block fixed point (four int4 digits per 32 values), v_dot8_i32_i4 against the 4-bit codes, i32 sums scaled and added in f32",
    "c2": "f32 in/out; x -> f16 (each row and K-slice scaled by a power of two), 4-bit codes x 6-bit scales as exact f16 integers, f16 MFMA with f32 accumulation, d / dmin and the K-slice sums in f32",
    "c3": "bf16 activations, weights dequantised (exact f32 value, one rounding) to a bf16 image by one pass, then a bf16 MFMA GEMM with f32 accumulation, f32 out",
    "c4": "f32 in/out; x -> 16-bit block fixed point (two int8 limbs per 32 values), v_dot4_i32_i8 against the 4-bit codes, i32 sums scaled (d * 6-bit scale, dmin * 6-bit minimum) and added in f32",
    "prefill": "f32 in/out; x and dequantised W rounded to f16 operands (x rows scaled by a power of two), f16 MFMA with f32 accumulation",
}
ARITHMETIC["ffn"] = ARITHMETIC["layer"] = ARITHMETIC["c4"]
DTYPE = {"c0": "int8 x int16 -> i32 dot, f32 accumulate", "c1": "int4 x int16 -> i32 dot, f32 accumulate",
         "c2": "f16 MFMA, f32 accumulate", "c3": "bf16 MFMA, f32 accumulate", "c4": "int4 x int16 -> i32 dot, f32 accumulate",
         "prefill": "f16 MFMA, f32 accumulate", "ffn": "int4 x int16 -> i32 dot, f32 accumulate", "layer": "int4 x int16 -> i32 dot, f32 accumulate"}


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--config", default="c4", choices=sorted(list(CONFIGS) + ["c4", "ffn", "layer"]))
    p.add_argument("--rows", type=int, default=1, help="activation rows of the ffn and layer workloads (a decode batch); default 1")
    p.add_argument("--no-others", action="store_true", help="measure the headline workload only")
    p.add_argument("--others", action="store_true", help="(default) also measure c0 .. c3; kept for older command lines")
    p.add_argument("--all", action="store_true", help="also measure prefill, ffn and layer")
    p.add_argument("--no-graph", action="store_true", help="submit the timed steps one call at a time")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    p.add_argument("--no-extras", action="store_true", help="skip the cache-resident pass, the plain-read yardstick and the clock sampling")
    p.add_argument("--ablation", default=None,
                   help="time a TIMING-ONLY variant of the fused GEMM (gemm_*: --config c3 with GOMLX_HIPQ_TWO_PASS_MIN_ROWS=100000, which sends C3 through that kernel), "
                        "of the Q4_K split-K route (q4k_*: --config c2) or of the decode GEMV (ks_*: --config c0) "
                        "instead of the product library (python -m gomlx_amd.ablate build NAME first): its results are wrong on purpose and the "
                        "line says so")
    p.add_argument("--hot", action="store_true", help="single weight buffer (Infinity-Cache resident) for the main measurement as well")
    p.add_argument("--copy-calibration", action="store_true",
                   help="instead of the benchmark, run a plain 64 MiB device-to-device copy kernel --steps times: the known-size "
                        "workload that hardware counter readings (FETCH_SIZE / WRITE_SIZE) are scaled by")
    p.add_argument("--yardstick", action="store_true",
                   help="instead of the benchmark, time the plain read-only kernel on 17.8 / 33.0 / 122.7 MB of cold weights")
    p.add_argument("--yardstick-size", choices=["c0", "c1", "c2", "c4"], default=None,
                   help="with --yardstick: only this workload's byte count, with ONE grid shape (--yardstick-shape), so that a "
                        "kernel trace of the run holds a single kind of launch")
    p.add_argument("--yardstick-shape", default=None,
                   help="workgroups,threads,depth of the read-only kernel for --yardstick-size (depth 100 + d: d non-temporal loads in "
                        "flight); default: the shape that usually reads that size fastest")
    p.add_argument("--matmul-yardstick", action="store_true",
                   help="instead of the benchmark, time the vendor library's plain bf16 GEMM (torch.matmul) on C3's shape, 2048 x 4096 x 4096: "
                        "what a 16-bit GEMM with no dequantisation reaches on this chip")
    p.add_argument("--l2-yardstick", action="store_true",
                   help="only measure how fast the L2 caches hand one small shared buffer to every workgroup (three access patterns)")
    p.add_argument("--mfma-valu-yardstick", action="store_true",
                   help="only measure how many vector-ALU instructions fit into the shadow of matrix instructions (cycles per group)")
    p.add_argument("--mfma-yardstick", action="store_true",
                   help="instead of the benchmark, time matrix instructions alone (the prefill GEMM's count and occupancy, no data movement) "
                        "with random and with zero operands and on a quarter of the CUs, with the shader clock the kernel measured itself")
    return p.parse_args()


# ---- HBM-side traffic per step, from hardware counters ------------------------------------------------------------
def measured_traffic(name):
    """Bytes per step from profiles/traffic.json: FETCH_SIZE and WRITE_SIZE (KiB per dispatch, summed over the step's
    kernels, one rocprofv3 --pmc run each), scaled by what the same counters read for the 64 MiB copy of
    --copy-calibration.  None when the file or the entry is missing (e.g. a kernel changed and was not re-profiled)."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            t = json.load(f)
        e, cal = t["workloads"][name], t["copy_calibration"]
        fs = cal["copied_kib"] / cal["fetch_size_kib"]
        ws = cal["copied_kib"] / cal["write_size_kib"]
        return int(round((e["fetch_size_kib"] * fs + e["write_size_kib"] * ws) * 1024))
    except (OSError, KeyError, ValueError, ZeroDivisionError):
        return None


# ---- clocks and power while a workload loops --------------------------------------------------------------------------
def _read(path):
    try:
        with open(path) as f:
            return f.read()
    except OSError:
        return None


def _active_mhz(text):
    if not text:
        return None
    for line in text.splitlines():
        if line.rstrip().endswith("*"):
            try:
                return float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
            except (IndexError, ValueError):
                return None
    return None


def sample_clock_state(busy_fn, seconds=0.25):
    """Runs busy_fn() in a loop for `seconds` and samples the first GPU's sysfs clock / power files from a second thread."""
    cards = sorted(glob.glob("/sys/class/drm/card[0-9]*/device/pp_dpm_sclk"))
    if not cards:
        return None
    dev = os.path.dirname(cards[0])
    power = sorted(glob.glob(os.path.join(dev, "hwmon", "hwmon*", "power1_average")) + glob.glob(os.path.join(dev, "hwmon", "hwmon*", "power1_input")))
    sclk, mclk, watts, stop = [], [], [], threading.Event()

    def sampler():
        while not stop.is_set():
            a, b = _active_mhz(_read(os.path.join(dev, "pp_dpm_sclk"))), _active_mhz(_read(os.path.join(dev, "pp_dpm_mclk")))
            if a:
                sclk.append(a)
            if b:
                mclk.append(b)
            if power:
                w = _read(power[0])
                try:
                    watts.append(float(w) / 1e6)
                except (TypeError, ValueError):
                    pass
            time.sleep(0.01)

    th = threading.Thread(target=sampler, daemon=True)
    th.start()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        busy_fn()
    stop.set()
    th.join()
    if not sclk and not mclk:
        return None
    med = lambda v: sorted(v)[len(v) // 2] if v else None
    return {"sclk_mhz": med(sclk), "sclk_mhz_min": min(sclk) if sclk else None, "mclk_mhz": med(mclk), "power_w": med(watts),
            "samples": len(sclk), "source": "sysfs pp_dpm_sclk / pp_dpm_mclk / hwmon power, sampled every 10 ms while the workload loops"}


# ---- the plain read-only kernel ---------------------------------------------------------------------------------------
class Yardstick:
    """gomlx_amd/libgq_yardstick.so: a kernel that loads every byte of a buffer once and does nothing else."""

    def __init__(self):
        path = os.path.join(ROOT, "gomlx_amd", "libgq_yardstick.so")
        self.lib = ctypes.CDLL(path)
        vp, i64 = ctypes.c_void_p, ctypes.c_int64
        self.lib.gqy_read.argtypes = [vp, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, i64, i64, ctypes.c_int, vp, vp]
        self.lib.gqy_read.restype = ctypes.c_int
        self.lib.gqy_mfma.argtypes = [vp, ctypes.c_int, ctypes.c_int, vp, vp, vp]
        self.lib.gqy_mfma.restype = ctypes.c_int

    # (workgroups, threads, loads in flight per thread): the shapes that read fastest on this chip at 18 .. 123 MB
    # (depth 100 + d: the same d loads in flight, issued as non-temporal loads)
    SHAPES = ((2048, 256, 2), (1024, 256, 4), (512, 256, 8), (256, 512, 8), (1024, 256, 104), (512, 256, 108))

    def time_buffers(self, torch, bufs, stream, tstream, steps, shapes=None):
        """Best mean time (us) per launch over SHAPES (or `shapes`): one recorded graph of `steps` launches rotating over `bufs`."""
        nbytes = bufs[0].numel() * bufs[0].element_size()
        out = torch.zeros(2048 * 512 + 16, dtype=torch.int32, device="cuda")
        best = None
        for wgs, threads, depth in shapes or self.SHAPES:
            def launch(i):
                rc = self.lib.gqy_read(bufs[i % len(bufs)].data_ptr(), nbytes, 0, wgs, threads, depth, 0, 0, 0, out.data_ptr(), stream)
                if rc:
                    raise RuntimeError(f"gqy_read failed ({rc})")
            for i in range(4):
                launch(i)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=tstream):
                for i in range(steps):
                    launch(i)
            with torch.cuda.stream(tstream):  # (a torch graph replays on the current stream)
                g.replay()
                torch.cuda.synchronize()
                for _ in range(3):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(tstream)
                    g.replay()
                    e1.record(tstream)
                    torch.cuda.synchronize()
                    us = e0.elapsed_time(e1) * 1e3 / steps
                    if best is None or us < best[0]:
                        best = (us, wgs, threads, depth)
            del g
        return best


_YARD = None


def yardstick():
    global _YARD
    if _YARD is None:
        try:
            _YARD = Yardstick()
        except OSError:
            _YARD = False
    return _YARD or None


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
        seed = workload_seed(name)
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
        self.use_copies = self.copies
        # one explicit stream for everything: warm-up, the recorded graph and the timed launches
        # (per-stream workspaces of the library must exist before a recording starts)
        self.tstream = torch.cuda.Stream()
        self.stream = self.tstream.cuda_stream
        torch.cuda.synchronize()

    def launch(self, step):
        c = step % self.use_copies
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

    def record(self, steps, first_step):
        L = self.L
        self.check(L.gq_graph_begin(self.stream))
        for s in range(steps):
            self.launch(first_step + s)
        g = ctypes.c_void_p()
        self.check(L.gq_graph_end(self.stream, ctypes.byref(g)))
        return g

    def run(self, steps, warmup, use_graph, extra_replays=2):
        """W untimed warm-up steps, then exactly K timed steps (the wall clock `value` is computed from); further
        replays of the same K steps only refine the kernel-time estimate."""
        torch, L = self.torch, self.L
        for s in range(warmup):
            self.launch(s)
        torch.cuda.synchronize()
        graph = None
        if use_graph:
            if warmup == 0:
                self.launch(0)  # creates the stream's workspace, if the path needs one
                torch.cuda.synchronize()
            graph = self.record(steps, warmup)
            if warmup > 0:  # untimed first replay: uploads the graph
                self.check(L.gq_graph_launch(graph, self.stream))
            torch.cuda.synchronize()

        def timed():
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
            return time.perf_counter() - t0, ev0.elapsed_time(ev1) * 1e3 / steps

        wall, region = timed()  # THE timed region: exactly K steps
        regions = [region]
        for _ in range(extra_replays if graph is not None else 0):
            regions.append(timed()[1])
        self.region_us_per_step = min(regions)
        self.graph = graph
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

    def rate(self, kernel_us):
        if self.bound == "hbm":
            return self.weight_bytes / (kernel_us * 1e-6) / 1e9, HBM_PEAK_GBS
        return self.flops / (kernel_us * 1e-6) / 1e12, MFMA_BF16_PEAK_TFLOPS

    def cache_resident(self, steps):
        """The same steps on a single weight buffer (everything but the largest workloads is then served from the
        Infinity Cache): not the metric, reported beside it."""
        torch, L = self.torch, self.L
        saved, self.use_copies = self.use_copies, 1
        try:
            for s in range(3):
                self.launch(s)
            torch.cuda.synchronize()
            g = self.record(steps, 0)
            self.check(L.gq_graph_launch(g, self.stream))
            torch.cuda.synchronize()
            best = None
            for _ in range(3):
                ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                ev0.record(self.tstream)
                self.check(L.gq_graph_launch(g, self.stream))
                ev1.record(self.tstream)
                torch.cuda.synchronize()
                us = ev0.elapsed_time(ev1) * 1e3 / steps
                best = us if best is None else min(best, us)
            self.check(L.gq_graph_destroy(g))
        finally:
            self.use_copies = saved
        ach, peak = self.rate(best)
        return {"kernel_us": best, "achieved": ach, "frac": ach / peak, "note": "single weight buffer: cache-resident, not the metric"}

    def plain_read(self, steps):
        """Time of the read-only kernel over the same cold bytes (concatenated weight copies of one step)."""
        ys = yardstick()
        if ys is None or self.bound != "hbm":
            return None
        torch = self.torch
        bufs = []
        for c in range(self.copies):
            parts = [p["W"][c].reshape(-1) for p in self.parts]
            bufs.append(parts[0] if len(parts) == 1 else torch.cat(parts))
        us, wgs, threads, depth = ys.time_buffers(torch, bufs, self.stream, self.tstream, max(10, min(steps, 50)))
        return {"us": us, "gbps": self.weight_bytes / us / 1e3, "frac_of_peak": self.weight_bytes / us / 1e3 / HBM_PEAK_GBS,
                "grid": f"{wgs} workgroups x {threads} threads, {depth % 100} {'non-temporal ' if depth >= 100 else ''}16-byte loads in flight per thread",
                "note": "read-only kernel over the same cold bytes, no arithmetic: what a one-shot kernel of this size can reach"}

    def clock_state(self):
        if getattr(self, "graph", None) is None:
            return None

        def busy():
            self.check(self.L.gq_graph_launch(self.graph, self.stream))
            self.torch.cuda.synchronize()
        return sample_clock_state(busy)

    def report(self, wall, kernel_us, steps):
        out = {}
        ach, peak = self.rate(kernel_us)
        if self.bound == "hbm":
            out["metric"], out["unit"] = "dense GEMV weight-GB/s", "GB/s"
            out["value"] = self.weight_bytes * steps / wall / 1e9
            out["roofline"] = {"bound": "hbm", "achieved": ach, "peak": peak, "unit": "GB/s",
                               "frac": ach / peak, "traffic": measured_traffic(self.name) if self.rows == 1 else None,
                               "algorithmic_bytes_per_launch": self.weight_bytes, "kernel_us": kernel_us}
        else:
            out["metric"], out["unit"] = "prefill GEMM TFLOP/s", "TFLOP/s"
            out["value"] = self.flops * steps / wall / 1e12
            out["roofline"] = {"bound": "mfma", "achieved": ach, "peak": peak, "unit": "TFLOP/s",
                               "frac": ach / peak, "traffic": measured_traffic(self.name),
                               "algorithmic_flops_per_launch": self.flops, "kernel_us": kernel_us}
        out["roofline"]["kernel_us_bracketed"] = self.bracketed_us_per_step
        out["roofline"]["kernel_us_region"] = self.region_us_per_step
        out["ms_per_step"] = wall / steps * 1e3
        return out

    def close(self):
        if getattr(self, "graph", None) is not None:
            self.check(self.L.gq_graph_destroy(self.graph))
            self.graph = None


def workload_seed(name):
    return 1000 + (int(name[1]) if name[0] == "c" else {"layer": 4, "ffn": 5, "prefill": 6}[name])


def host_threads():
    """Threads for the CPU baseline: the CPUs this process may run on, within the share the box grants a one-GPU job
    (it exports OMP_NUM_THREADS for that)."""
    try:
        n = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        n = os.cpu_count() or 1
    try:
        cap = int(os.environ.get("OMP_NUM_THREADS", "0"))
    except ValueError:
        cap = 0
    return max(1, min(n, cap) if cap > 0 else n)


def reference_toolchain():
    """Whether the reference's own CPU backend could be timed on this host: a Go toolchain and a module cache that holds
    github.com/gomlx/compute v0.1.2 (go.mod:10 of the reference).  Looked for, never fetched or built."""
    import shutil
    go = shutil.which("go")
    info = {"go": go, "go_version": None, "gomlx_compute_v0.1.2_in_module_cache": False}
    if go:
        try:
            import subprocess
            info["go_version"] = subprocess.run([go, "version"], capture_output=True, text=True, timeout=20).stdout.strip() or None
        except (OSError, subprocess.SubprocessError):
            pass
    roots = [os.environ.get("GOMODCACHE")]
    roots += [os.path.join(g, "pkg", "mod") for g in (os.environ.get("GOPATH") or os.path.join(os.path.expanduser("~"), "go")).split(os.pathsep) if g]
    for r in roots:
        if r and os.path.isdir(os.path.join(r, "github.com", "gomlx", "compute@v0.1.2")):
            info["gomlx_compute_v0.1.2_in_module_cache"] = True
    info["usable"] = bool(go) and info["gomlx_compute_v0.1.2_in_module_cache"]
    if not info["usable"]:
        info["consequence"] = "the reference's Go backend cannot be run here: the baseline is this repository's C restatement of its algorithm (kind: port)"
    return info


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return None


def cpu_baseline(name, min_runs=5, min_seconds=3.0, max_seconds=25.0):
    """The CPU oracle's fused fp32 restatement on the host cores (checker code used as a reported baseline only), on the
    inputs the GPU leg uses (same seeds): >= 2 warm-ups, then >= 5 runs and >= 3 s, like the reference's own timing
    protocol (internal/perf/dotgeneral_perf_test.go:366-381), capped at ~25 s (the side workloads: 1 warm-up, >= 3 runs and
    >= 1.5 s, so that the default run stays within minutes)."""
    from gomlx_amd import ggml, synth
    from oracle import ggml_oracle as oracle
    cores = host_threads()
    if name in ("c4", "layer"):
        shapes = [("Q4_K", 1, K, N) for K, N in C4_SHAPES]
    elif name == "ffn":  # the two projections; the normalisation and the product are negligible beside them
        shapes = [("Q4_K", 1, 4096, 14336)] * 2
    else:
        tn, M, K, N, _, _ = CONFIGS[name]
        shapes = [(tn, M, K, N)]
    sample = "full workload"
    rows = None
    if name in ("c3", "prefill"):  # 34 GMAC per pass is minutes of CPU time: the first 64 of the 2048 activation rows
        rows = 64
        sample = "the first 64 of the 2048 activation rows (1/32 of the FLOPs), all of W"
    seed = workload_seed(name)
    probs = []
    for i, (tn, M, K, N) in enumerate(shapes):
        t = getattr(ggml, tn)
        x = synth.activations(seed + 100 + i, M, K)
        if rows:
            x = x[:rows]
        if name == "c3":
            import torch
            x = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
        probs.append((t, x, synth.weights(t, seed + i, N, K)))
    wbytes = sum(p[2].size for p in probs)
    flops = sum(2 * p[1].shape[0] * p[1].shape[1] * p[2].shape[0] for p in probs)

    def once():
        for t, x, W in probs:
            oracle.c_qdense(t, x, W, None, 0, f32acc_threads=cores)

    once()
    if min_runs >= 5:
        once()
    runs, t0 = 0, time.perf_counter()
    while True:
        once()
        runs += 1
        el = time.perf_counter() - t0
        if (runs >= min_runs and el >= min_seconds) or el >= max_seconds:
            break
    per = el / runs
    common = {"cores": cores, "host_cpus": os.cpu_count(), "cpu_model": cpu_model(), "kind": "port",
              "sample": f"{sample}, same seeded inputs as the GPU leg; {runs} runs, {per * 1e3:.2f} ms each; OpenMP over output rows"}
    if name in ("c3", "prefill"):
        return {"value": flops / per / 1e12, "unit": "TFLOP/s", **common}
    return {"value": wbytes / per / 1e9, "unit": "GB/s", **common}


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


YARDSTICK_BYTES = {"c0": 17825792, "c1": 33030144, "c2": 33030144, "c4": 122683392}
YARDSTICK_DEFAULT_SHAPE = {"c0": (512, 256, 108), "c1": (1024, 256, 104), "c2": (1024, 256, 104), "c4": (256, 512, 8)}


def yardstick_only(torch, steps, size=None, shape=None):
    """The plain read-only kernel on cold buffers of the decode workloads' sizes (best of several grid shapes), or, with
    `size`, on that one size with one grid shape (for a kernel trace that holds a single kind of launch)."""
    ys = yardstick()
    if ys is None:
        print("bench.py: gomlx_amd/libgq_yardstick.so is missing (python -m gomlx_amd.build)", file=sys.stderr)
        sys.exit(4)
    tstream = torch.cuda.Stream()
    out = {"yardstick": "read-only kernel, every byte loaded once, no arithmetic; cold: rotation over > 512 MB of distinct buffers", "sizes": {}}
    shapes = None
    if size is not None:
        shapes = (tuple(int(v) for v in shape.split(",")) if shape else YARDSTICK_DEFAULT_SHAPE[size],)
        if len(shapes[0]) != 3:
            print("bench.py: --yardstick-shape wants workgroups,threads,depth", file=sys.stderr)
            sys.exit(2)
    for name, nbytes in YARDSTICK_BYTES.items():
        if size is not None and name != size:
            continue
        copies = max(2, -(-(512 << 20) // nbytes) + 1)
        bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda") for _ in range(copies)]
        us, wgs, threads, depth = ys.time_buffers(torch, bufs, tstream.cuda_stream, tstream, steps, shapes)
        out["sizes"][name] = {"bytes": nbytes, "us": us, "gbps": nbytes / us / 1e3, "frac_of_peak": nbytes / us / 1e3 / HBM_PEAK_GBS,
                              "grid": f"{wgs} x {threads}, depth {depth}", "copies": copies}
        del bufs
        torch.cuda.empty_cache()
    print(json.dumps(out))


def matmul_yardstick(torch, steps):
    """torch.matmul in bf16 on C3's shape (x [2048, 4096] . W^T, W [4096, 4096] already a 16-bit matrix), fp32 result via a bf16
    output widened afterwards is NOT included: the vendor kernel writes bf16, half the output bytes of this library's fp32."""
    M, K, N = 2048, 4096, 4096
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    ws = [torch.randn(N, K, device="cuda").to(torch.bfloat16) for _ in range(17)]  # > 512 MB: cold, like the benchmark's rotation
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        for i in range(5):
            torch.matmul(x, ws[i % len(ws)].t())
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(st)
            for i in range(steps):
                torch.matmul(x, ws[i % len(ws)].t())
            e1.record(st)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / steps
            best = us if best is None else min(best, us)
    flops = 2.0 * M * K * N
    return {"matmul_yardstick": "torch.matmul bf16 [2048,4096] x [4096,4096]^T, bf16 output, cold weights", "us": best,
            "tflops": flops / best / 1e6, "frac_of_peak": flops / best / 1e6 / MFMA_BF16_PEAK_TFLOPS, "steps": steps}


def mfma_yardstick(torch, steps, only_first=False):
    """Matrix instructions only (gomlx_amd/csrc/yardstick.hip, gqy_mfma): the prefill GEMM's instruction count per wavefront
    (64 K-steps x 16 v_mfma_f32_32x32x16_bf16) and its occupancy (8 wavefronts per CU), no data movement at all.  Reported per
    case: time per launch (HIP events over `steps` back-to-back launches), the rate that corresponds to, and the shader clock
    the workgroups measured themselves (clock counter over the constant 100 MHz counter)."""
    ys = yardstick()
    if ys is None:
        return None
    groups, cus = 64 * 4, torch.cuda.get_device_properties(0).multi_processor_count
    st = torch.cuda.Stream()
    out = {"mfma_yardstick": "v_mfma_f32_32x32x16_bf16 only: 1024 per wavefront, 8 wavefronts per workgroup, no loads, LDS or barriers in the loop",
           "published_peak_tflops": MFMA_BF16_PEAK_TFLOPS, "cases": {}}
    sink = torch.zeros(cus * 512, device="cuda")
    cases = (("random operands, one workgroup per CU", "randn", cus), ("zero operands, one workgroup per CU", "zeros", cus),
             ("random operands, a quarter of the CUs", "randn", cus // 4))
    for label, fill, wgs in cases[:1] if only_first else cases:
        frags = (torch.randn(8 * 4 * 64 * 8, device="cuda") if fill == "randn" else torch.zeros(8 * 4 * 64 * 8, device="cuda")).to(torch.bfloat16)
        clocks = torch.zeros(4 * wgs, dtype=torch.int64, device="cuda")

        def launch():
            rc = ys.lib.gqy_mfma(frags.data_ptr(), groups, wgs, clocks.data_ptr(), sink.data_ptr(), st.cuda_stream)
            if rc:
                raise RuntimeError(f"gqy_mfma failed ({rc})")
        with torch.cuda.stream(st):
            for _ in range(5):
                launch()
            torch.cuda.synchronize()
            best = None
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(st)
                for _ in range(steps):
                    launch()
                e1.record(st)
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) * 1e3 / steps
                best = us if best is None else min(best, us)
        c = clocks.cpu().view(wgs, 4).double()
        loop_us = (c[:, 3] - c[:, 1]) / 100.0
        mhz = (c[:, 2] - c[:, 0]) / loop_us
        flops = wgs * 8 * 4 * groups * 2.0 * 32 * 32 * 16
        out["cases"][label] = {"workgroups": wgs, "us_per_launch": best, "tflops": flops / best / 1e6,
                               "frac_of_published_peak": flops / best / 1e6 / (MFMA_BF16_PEAK_TFLOPS * wgs / cus),
                               "shader_mhz_mean": float(mhz.mean()), "shader_mhz_min": float(mhz.min()),
                               "wavefront0_loop_us_mean": float(loop_us.mean())}
    return out


def l2_yardstick(torch, steps=50):
    """How fast the L2 caches hand ONE small buffer to every workgroup at once (gomlx_amd/csrc/yardstick.hip, gqy_read_shared /
    gqy_read_streams): what a small-batch kernel pays that streams the whole activation image (0.9 MB of fp16 fragments for 32
    columns at K = 14336) past every workgroup instead of splitting K.  Three ways to read 56 records of 16 KiB in each of 256
    workgroups of 512 threads: the workgroup walks the buffer together; every wavefront walks its own records (w, w + 8, ...) with
    ordinary loads, 16 KiB in flight per wavefront; the same by LDS DMA through a ring of four 4 KiB slots per wavefront (12 KiB
    in flight).  HIP events around `steps` launches."""
    ys = yardstick()
    if ys is None:
        return None
    vp = ctypes.c_void_p
    ys.lib.gqy_read_streams.argtypes = [vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp]
    ys.lib.gqy_read_streams.restype = ctypes.c_int
    ys.lib.gqy_read_shared.argtypes = [vp, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp]
    ys.lib.gqy_read_shared.restype = ctypes.c_int
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    st = torch.cuda.Stream()
    sink = torch.zeros(2048 * 1024, dtype=torch.int32, device="cuda")
    records, rec = 56, 16384
    buf = torch.randint(0, 255, (records * rec,), dtype=torch.uint8, device="cuda")
    cases = {
        "workgroup walks the buffer together (ordinary loads, 8 per thread in flight)":
            lambda: ys.lib.gqy_read_shared(buf.data_ptr(), records * rec, cus, 512, 1, sink.data_ptr(), st.cuda_stream),
        "one stream of records per wavefront, ordinary loads (16 KiB in flight per wavefront)":
            lambda: ys.lib.gqy_read_streams(buf.data_ptr(), records, rec, cus, 0, sink.data_ptr(), st.cuda_stream),
        "one stream of records per wavefront, LDS DMA ring (12 KiB in flight per wavefront)":
            lambda: ys.lib.gqy_read_streams(buf.data_ptr(), records, rec, cus, 1, sink.data_ptr(), st.cuda_stream),
    }
    out = {"l2_yardstick": f"{cus} workgroups x 512 threads each read the same {records * rec} bytes", "cases": {}}
    total = records * rec * cus
    for label, fn in cases.items():
        with torch.cuda.stream(st):
            for _ in range(3):
                if fn():
                    raise RuntimeError("yardstick launch failed")
            torch.cuda.synchronize()
            best = None
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(st)
                for _ in range(steps):
                    fn()
                e1.record(st)
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) * 1e3 / steps
                best = us if best is None else min(best, us)
        out["cases"][label] = {"us_per_launch": best, "tb_per_s_out_of_l2": total / best / 1e6, "bytes_per_clock_per_cu_at_2400mhz": total / cus / best / 2400.0}
    return out


def mfma_valu_yardstick(torch, groups=512):
    """Vector-ALU instructions in the shadow of matrix instructions (gomlx_amd/csrc/yardstick.hip, gqy_mfma_valu): shader cycles
    per group of four independent v_mfma_f32_32x32x16_bf16 per wavefront plus NV independent vector-ALU instructions, placed
    behind the group or NV / 4 behind each matrix instruction, accumulators in ordinary or in accumulation registers, for one
    and two wavefronts per SIMD (128 resp. 256 cycles of matrix work per group), on one workgroup (no power limit in play) and on
    one workgroup per CU.  Cycles: shader clock counter, from the first wavefront's start to the last one's end, per workgroup,
    mean over workgroups.  A figure that stays at the matrix cycles means the vector-ALU work is free; 4 more cycles per
    instruction and wavefront mean that nothing overlaps."""
    ys = yardstick()
    if ys is None:
        return None
    vp = ctypes.c_void_p
    ys.lib.gqy_mfma_valu.argtypes = [vp] + [ctypes.c_int] * 7 + [vp, vp, vp]
    ys.lib.gqy_mfma_valu.restype = ctypes.c_int
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    st = torch.cuda.Stream()
    frags = torch.randn(8 * 4 * 64 * 8, device="cuda").to(torch.bfloat16)
    sink = torch.zeros(cus * 512, device="cuda")
    kinds = {0: "v_fma_f32", 1: "v_xor_b32", 2: "v_cvt_pk_bf16_f32"}
    out = {"mfma_valu_yardstick": "shader cycles per group of 4 x v_mfma_f32_32x32x16_bf16 + NV independent vector-ALU instructions per wavefront",
           "groups_per_wavefront": groups, "rows": []}
    for wgs in (1, cus):
        for threads in (256, 512):
            for acc in (0, 1):
                for kind in (0, 1, 2):
                    for place in (0, 1):
                        waves = threads // 64
                        row = {"workgroups": wgs, "wavefronts_per_simd": threads // 256, "matrix_cycles_per_group": 128 * (threads // 256),
                               "accumulators": "accumulation registers" if acc else "ordinary registers", "instruction": kinds[kind],
                               "placement": "interleaved" if place else "behind the group", "cycles_per_group": {}, "shader_mhz": {}}
                        for nv in (0, 8, 16, 32, 48):
                            clocks = torch.zeros(32 * wgs, dtype=torch.int64, device="cuda")
                            with torch.cuda.stream(st):
                                for _ in range(3):  # (the last launch's stamps are the ones read)
                                    rc = ys.lib.gqy_mfma_valu(frags.data_ptr(), groups, wgs, threads, nv, place, kind, acc, clocks.data_ptr(),
                                                              sink.data_ptr(), st.cuda_stream)
                                    if rc:
                                        raise RuntimeError(f"gqy_mfma_valu failed ({rc})")
                                torch.cuda.synchronize()
                            c = clocks.cpu().view(wgs, 8, 4)[:, :waves, :].double()
                            span = c[:, :, 2].max(dim=1).values - c[:, :, 0].min(dim=1).values
                            wall = (c[:, :, 3].max(dim=1).values - c[:, :, 1].min(dim=1).values) / 100.0
                            row["cycles_per_group"][str(nv)] = round(float((span / groups).mean()), 1)
                            row["shader_mhz"][str(nv)] = round(float((span / wall).mean()))
                        out["rows"].append(row)
    return out


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
    if args.yardstick:
        yardstick_only(torch, min(args.steps, 50), args.yardstick_size, args.yardstick_shape)
        return
    if args.matmul_yardstick:
        print(json.dumps(matmul_yardstick(torch, min(args.steps, 50))))
        return
    if args.l2_yardstick:
        out = l2_yardstick(torch)
        if out is None:
            print("bench.py: gomlx_amd/libgq_yardstick.so is missing (python -m gomlx_amd.build)", file=sys.stderr)
            sys.exit(4)
        print(json.dumps(out))
        return
    if args.mfma_valu_yardstick:
        out = mfma_valu_yardstick(torch)
        if out is None:
            print("bench.py: gomlx_amd/libgq_yardstick.so is missing (python -m gomlx_amd.build)", file=sys.stderr)
            sys.exit(4)
        print(json.dumps(out))
        return
    if args.mfma_yardstick:
        out = mfma_yardstick(torch, min(args.steps, 200))
        if out is None:
            print("bench.py: gomlx_amd/libgq_yardstick.so is missing (python -m gomlx_amd.build)", file=sys.stderr)
            sys.exit(4)
        print(json.dumps(out))
        return
    from gomlx_amd import _lib
    if args.ablation:
        from gomlx_amd import ablate
        if args.ablation not in ablate.VARIANTS or not os.path.exists(ablate.lib_path(args.ablation)):
            print(f"bench.py: no built ablation {args.ablation!r}: python -m gomlx_amd.ablate build [{' | '.join(ablate.VARIANTS)}]", file=sys.stderr)
            sys.exit(4)
        _lib.use_library(ablate.lib_path(args.ablation))
    _lib.init(0)

    def measure(name, steps):
        prob = Problem(torch, name, hot=args.hot, rows=args.rows)
        wall, kus, launches = prob.run(steps, args.warmup, not args.no_graph)
        rep = prob.report(wall, kus, steps)
        rep["weight_copies"] = prob.copies
        rep["launches_per_step"] = launches
        if not args.no_extras:
            if not args.hot:
                rep["roofline"]["cache_resident"] = prob.cache_resident(steps)
            pr = prob.plain_read(steps)
            if pr is not None:
                pr["kernel_over_plain_read"] = rep["roofline"]["kernel_us"] / pr["us"]
                rep["roofline"]["plain_read"] = pr
            rep["clock_state"] = prob.clock_state()
        bound = prob.bound
        prob.close()
        del prob
        torch.cuda.empty_cache()
        if not args.no_extras and bound == "mfma":
            # measured in the same process right after the workload: the vendor library's plain bf16 GEMM on the same shape
            # (no dequantisation, bf16 result) and the matrix instructions of such a GEMM alone
            ku = rep["roofline"]["kernel_us"]
            vg = matmul_yardstick(torch, 30)
            rep["roofline"]["vendor_gemm"] = {"us": vg["us"], "tflops": vg["tflops"], "kernel_over_vendor_gemm": ku / vg["us"],
                                              "note": "torch.matmul bf16 2048 x 4096 x 4096, weights already 16-bit, bf16 result, same run"}
            torch.cuda.empty_cache()
            mo = mfma_yardstick(torch, 100, only_first=True)
            if mo is not None:
                c = next(iter(mo["cases"].values()))
                rep["roofline"]["mfma_only"] = {"us": c["us_per_launch"], "tflops": c["tflops"], "shader_mhz": c["shader_mhz_mean"],
                                                "kernel_over_mfma_only": ku / c["us_per_launch"],
                                                "note": "the same number of v_mfma_f32_32x32x16_bf16 per wavefront at the same occupancy and "
                                                        "nothing else (random operands): what the chip sustains under its power limit"}
        return rep

    rep = measure(args.config, args.steps)
    tn = "Q4_K" if args.config in ("c4", "ffn", "layer") else CONFIGS[args.config][0]
    line = {
        "metric": rep["metric"], "value": rep["value"], "unit": rep["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": rep["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": DTYPE[args.config], "data": "synthetic",
        "config": {"workload": WORKLOAD_TEXT[args.config] + (f" [run with {args.rows} activation rows]" if args.rows != 1 and args.config in ("ffn", "layer") else ""),
                   "ggml_type": tn,
                   "arithmetic": ARITHMETIC[args.config],
                   "weights": "cache-resident single buffer" if args.hot else
                   f"cold: rotation over {rep['weight_copies']} distinct weight copies",
                   "submission": "eager" if args.no_graph else "one recorded HIP graph of all timed steps",
                   "launches_per_step": rep["launches_per_step"]},
        "roofline": rep["roofline"],
        "clock_state": rep.get("clock_state"),
    }
    if args.ablation:
        from gomlx_amd import ablate
        line["ablation"] = {"name": args.ablation, "taken_out": ablate.VARIANTS[args.ablation][1],
                            "note": "TIMING ONLY: this library computes wrong results on purpose; the line is not a benchmark result"}
        line["metric"] = "ablation timing (not a result): " + line["metric"]
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(args.config)
        line["cpu_baseline"]["reference_toolchain"] = reference_toolchain()
    if not args.no_others:
        names = ["c0", "c1", "c2", "c3", "c4"] + (["prefill", "ffn", "layer"] if args.all else [])
        others = {}
        for name in names:
            if name == args.config:
                continue
            # (the side measurements choose their own step counts: --steps is the headline's; short runs of the small
            # workloads read up to 10 % slow)
            steps = max(args.steps, 200) if name not in ("c3", "prefill") else max(30, args.steps // 10)
            r = measure(name, steps)
            others[name] = {"workload": WORKLOAD_TEXT[name], "dtype": DTYPE[name], "arithmetic": ARITHMETIC[name], "metric": r["metric"],
                            "value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"], "roofline": r["roofline"],
                            "clock_state": r.get("clock_state"), "steps": steps, "launches_per_step": r["launches_per_step"]}
            if not args.no_cpu and name in ("c0", "c1", "c2", "c3", "c4"):  # the five benchmark configurations each carry their CPU baseline
                others[name]["cpu_baseline"] = cpu_baseline(name, min_runs=3, min_seconds=1.5, max_seconds=12.0)
        line["others"] = others
    print(json.dumps(line))


if __name__ == "__main__":
    main()
