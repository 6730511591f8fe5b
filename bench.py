#!/usr/bin/env python3
"""Benchmark of the batch-1 fused trellis decode + mat-vec on one MI355X.

One step = one call of decompress_matvec_16_8_1 (hashed-codebook stream, 2 bits/weight, 16-bit
window) on the Llama-2-7B down-projection shape m=4096, n=11008, batch 1, through the C ABI.
Steps rotate over distinct weight copies whose total is at least 600 MB (more than twice the 256 MB
Infinity Cache) whatever --steps is, and the caches are flushed with a 1 GiB read-modify-write pass between
the untimed and the timed replay, so every timed launch streams its weights from HBM.  The metric is GB/s
of compressed weight bytes.

The line printed at the end also carries
  roofline      compressed bytes per launch / average launch duration (HIP events on the launch
                stream over the timed region) against the 8 TB/s HBM peak;
  cpu_baseline  the CPU oracle's fused decode+mat-vec (the checker, timed here only as a
                baseline) on the host cores of the same box.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "let-it-slide_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0



def measured_traffic(kernel, m, n):
    """HBM bytes per launch (per layer for a chain kernel) of `kernel` on an m x n layer, as measured with
    `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` on `bench.py --pmc-probe` and written down in
    profiles/<kernel>_<m>x<n>.md (lines `traffic_bytes = N` and `measured_at = <commit>`).  The figure is a property of the
    kernel that file names at that commit, not of this run: (None, None) when there is no such summary."""
    import re
    path = os.path.join(ROOT, "profiles", f"{kernel}_{m}x{n}.md")
    if not os.path.exists(path):
        return None, None
    text = open(path).read()
    t = re.search(r"^traffic_bytes\s*=\s*([\d,]+)", text, flags=re.M)
    c = re.search(r"^measured_at\s*=\s*(\w+)", text, flags=re.M)
    return (int(t.group(1).replace(",", "")) if t else None), (c.group(1) if c else None)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--copies", type=int, default=0,
                    help="distinct weight copies to rotate over (0: as many as make 600 MB, at least 32)")
    ap.add_argument("--m", type=int, default=4096)
    ap.add_argument("--n", type=int, default=11008)
    ap.add_argument("--S", type=int, default=8, choices=(6, 8))
    ap.add_argument("--launch", choices=("chain", "graph", "direct"), default="chain",
                    help="chain: the timed steps are the layers of ONE rptc_decompress_matvec_chain launch (the per-launch "
                         "figure is reported beside it); graph: one launch per step, captured in a HIP graph; "
                         "direct: one host call per step")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="for `rocprofv3 --pmc`: a few direct launches of the kernel, of the chain, of the transposed "
                         "mat-vec and of the batch-16 product, plus a plain device copy of known size (the calibration "
                         "for FETCH_SIZE / WRITE_SIZE); prints no benchmark line")
    ap.add_argument("--extra-shapes", action="store_true", help="also time the other layer shapes")
    ap.add_argument("--other-ops", action="store_true",
                    help="time decompress, decompress_matvec_t_16 and sign_hadamard instead (prints its own JSON line)")
    ap.add_argument("--quantize", action="store_true", help="time the Viterbi search kernel of the quantizer")
    ap.add_argument("--decode", action="store_true",
                    help="greedy decode with a Llama-2-7B-shaped random-init model whose projections are 2-bit streams "
                         "(prompt 512, 128 new tokens, batch 1); prints its own JSON line")
    ap.add_argument("--decode-layers", type=int, default=32)
    ap.add_argument("--decode-quantized", action="store_true",
                    help="with --decode: the projections are random-init dense weights put through the quantizer "
                         "(row/column factorisation + trellis search) instead of random streams; their scales and "
                         "biases are applied inside the mat-vec kernels")
    ap.add_argument("--valu-probe", action="store_true",
                    help="issue rate of the vector instructions the decode consists of (four waves a SIMD, registers only)")
    ap.add_argument("--matmul", action="store_true",
                    help="time the batch 8/16/32 fused decode + MFMA mat-mat instead (prints its own JSON line)")
    return ap.parse_args()


COLD_SET_BYTES = 600 << 20      # the rotating copies add up to at least this: > 2 x the 256 MB Infinity Cache


def cold_copies(asked, layer_bytes):
    """Copies to rotate over: what was asked for, but never fewer than make COLD_SET_BYTES (so that a copy is
    revisited only after more than two cache sizes of other data), and at least 32."""
    need = max(32, -(-COLD_SET_BYTES // layer_bytes))
    return max(asked, need)


_evict_buffer = None


def evict_caches():
    """A read-modify-write pass over 1 GiB: whatever the L2s and the Infinity Cache held is gone afterwards."""
    import torch
    global _evict_buffer
    if _evict_buffer is None:
        _evict_buffer = torch.zeros(1 << 28, dtype=torch.int32, device="cuda")
    _evict_buffer.add_(1)
    torch.cuda.synchronize()


def aids_library():
    """bench_aids/librptc_bench_aids.so: an empty launch, read-only kernels, instruction issue rates (measurement aids,
    not the product)."""
    path = os.path.join(ROOT, "bench_aids", "librptc_bench_aids.so")
    lib = ctypes.CDLL(path)
    lib.rptc_probe_read_chain.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p,
                                          ctypes.c_void_p]
    lib.rptc_probe_lds.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.rptc_probe_empty.argtypes = [ctypes.c_int, ctypes.c_void_p]
    lib.rptc_probe_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
    lib.rptc_probe_valu.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.rptc_probe_decode.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    return lib


class Runner:
    """Launches the op through the C ABI with pre-bound arguments (no timing, asynchronous)."""

    def __init__(self, m, n, S, copies, seed=42, bits=2):
        import torch
        import rptc_kernels
        self.torch = torch
        self.m, self.n, self.S = m, n, S
        self.lib = rptc_kernels.library()
        rc = self.lib.rptc_init()
        if rc:
            raise RuntimeError(self.lib.rptc_status_string(rc).decode())
        self.bits = bits
        self.fn = getattr(self.lib, f"rptc_decompress_matvec_16_{S}_1") if bits == 2 else None
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        words = m * n * bits // 32
        self.weights = [torch.randint(-(1 << 31), 1 << 31, (words,), generator=g, dtype=torch.int64,
                                      device="cuda").to(torch.int32) for _ in range(copies)]
        self.codebook = torch.randn(2 << S, generator=g, device="cuda").to(torch.float16)
        self.x = torch.randn(n, generator=g, device="cuda").to(torch.float16)
        self.out = torch.zeros(m, dtype=torch.float16, device="cuda")
        self.bytes = m * n * bits // 8
        torch.cuda.synchronize()

    def launch(self, k, stream):
        w = self.weights[k % len(self.weights)]
        if self.bits == 2:
            rc = self.fn(w.data_ptr(), self.codebook.data_ptr(), self.x.data_ptr(), self.out.data_ptr(),
                         self.m, self.n, 0, ctypes.c_void_p(stream), None)
        else:
            rc = self.lib.rptc_decompress_matvec_bits(w.data_ptr(), self.codebook.data_ptr(), self.x.data_ptr(),
                                                      self.out.data_ptr(), self.m, self.n, self.S, self.bits, 0,
                                                      ctypes.c_void_p(stream), None)
        if rc:
            raise RuntimeError(self.lib.rptc_status_string(rc).decode())

    def run(self, steps, warmup, mode):
        """Returns (wall seconds, event milliseconds) for exactly `steps` launches."""
        torch = self.torch
        stream = torch.cuda.current_stream()
        for k in range(warmup):
            self.launch(k, stream.cuda_stream)
        torch.cuda.synchronize()
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        if mode == "graph":
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                cs = torch.cuda.current_stream().cuda_stream
                for k in range(steps):
                    self.launch(k, cs)
            graph.replay()                      # untimed: first replay uploads the graph
            torch.cuda.synchronize()
            evict_caches()                      # the timed replay starts with cold caches
            t0 = time.perf_counter()
            ev0.record()
            graph.replay()
            ev1.record()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
        else:
            evict_caches()
            t0 = time.perf_counter()
            ev0.record()
            for k in range(steps):
                self.launch(k, stream.cuda_stream)
            ev1.record()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
        return t1 - t0, ev0.elapsed_time(ev1)

    def chain_run(self, steps, warmup):
        """`steps` layers (step k = weight copy k % copies, an output of its own per step: layers that write one buffer
        depend on each other, and such a chain is run as separate launches) as ONE chain launch.
        Returns (wall seconds, event milliseconds, rel-L2 of the last layer's output against the dense product)."""
        torch = self.torch
        import rptc_kernels
        copies = len(self.weights)
        outs = torch.zeros((max(steps, warmup, 1), self.m), dtype=torch.float16, device="cuda")
        chain = rptc_kernels.MatvecChain([(self.weights[k % copies], self.x, outs[k]) for k in range(steps)], self.codebook)
        warm = rptc_kernels.MatvecChain([(self.weights[k % copies], self.x, outs[k]) for k in range(max(warmup, 1))],
                                        self.codebook)
        warm.run(carry_mode=0, timed=False)
        # one untimed launch of the chain itself, as the graph of the per-launch pattern is replayed once before it is
        # timed: the first long launch after the set-up work runs at clocks that are still rising (5.9 us a layer
        # against 5.0-5.4 for every later one)
        chain.run(carry_mode=0, timed=False)
        torch.cuda.synchronize()
        evict_caches()
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record()
        chain.run(carry_mode=0, timed=False)
        ev1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        if not chain.one_launch:
            raise RuntimeError("the chain was not planned as one launch")
        W = torch.zeros((self.m, self.n), dtype=torch.float16, device="cuda")
        rptc_kernels.matvec_bits_dense(self.weights[(steps - 1) % copies], self.codebook, W, 2)
        want = W.double() @ self.x.double()
        err = ((outs[steps - 1].double() - want).norm() / want.norm()).item()
        if not err < 1e-3:
            raise RuntimeError(f"chain output is wrong: rel-L2 {err}")
        return t1 - t0, ev0.elapsed_time(ev1), err

    def check(self):
        """Guard against timing a kernel that computes nothing: the output must equal the dense
        product of the exported matrix (full parity lives in tests/)."""
        torch = self.torch
        import rptc_kernels
        W = torch.zeros((self.m, self.n), dtype=torch.float16, device="cuda")
        rptc_kernels.matvec_bits_dense(self.weights[0], self.codebook, W, self.bits)
        self.launch(0, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        want = W.double() @ self.x.double()
        err = ((self.out.double() - want).norm() / want.norm()).item()
        if not err < 1e-3:
            raise RuntimeError(f"kernel output is wrong: rel-L2 {err}")
        return err


def cpu_baseline(runner, min_seconds=8.0, also_seconds=4.0):
    """The oracle's fused decode + mat-vec (fp32 accumulate, threads over rows) on the same layer, repeated until it has
    run for min_seconds; and, under "also", the same on the 4096 x 4096 layer (the single-layer configuration the
    reference's own CPU path would run) for also_seconds."""
    import numpy as np
    from oracle import rptc_oracle
    threads = rptc_oracle.num_threads()

    def timed(comp, cb, x, m, n, S, seconds):
        rptc_oracle.matvec_f32(comp, cb, x, m, S)                     # warm the caches and the thread pool
        reps, t0 = 0, time.perf_counter()
        while True:
            rptc_oracle.matvec_f32(comp, cb, x, m, S)
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= seconds and reps >= 3:
                break
        return {"value": round(m * n // 4 * reps / dt / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": f"{reps} full passes of the same {m}x{n} layer, {dt:.1f} s of CPU work", "ms_per_pass": round(dt / reps * 1e3, 3)}

    cb = runner.codebook.cpu().numpy()
    out = timed(runner.weights[0].cpu().numpy().view(np.uint32), cb, runner.x.cpu().numpy(), runner.m, runner.n, runner.S, min_seconds)
    if (runner.m, runner.n) != (4096, 4096) and also_seconds > 0:
        rng = np.random.default_rng(42)
        comp = rng.integers(0, 1 << 32, 4096 * 4096 // 16, dtype=np.uint64).astype(np.uint32)
        x = rng.standard_normal(4096).astype(np.float16)
        out["also"] = {"4096x4096": timed(comp, cb, x, 4096, 4096, runner.S, also_seconds)}
    return out


MFMA_F16_PEAK_TFLOPS = 2516.6


# HBM traffic of the batch-16 product on 4096 x 11008 (same --pmc-probe runs as above): 14 071 KiB read (stream,
# partial tiles read back, packed activations) + 1 683 KiB written (partial tiles, packed activations, output)
MEASURED_MATMUL_TRAFFIC_BYTES = {(4096, 11008, 8, 16, 2): 16132000}


def _hbm_roofline(stream_bytes, us, traffic=None):
    """The roofline object of a stream-bound call: its algorithmic bytes are the compressed stream (the layers are at
    128-256 flop/byte at batch 16-32, below the 315 flop/byte ridge of fp16 MFMA over HBM)."""
    gbs = stream_bytes / us / 1e3
    return {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic}


def bench_matmul(a):
    """Batch 8/16/32 fused decode + mat-mat on the same layer, next to decode-then-dense-GEMM
    (dense export kernel + torch.matmul on the decoded fp16 matrix) and to the batch-1 mat-vec on the same stream."""
    import torch
    import rptc_kernels
    lib = rptc_kernels.library()
    rptc_kernels.set_timing(False)
    m, n, S = a.m, a.n, a.S
    g = torch.Generator(device="cuda")
    g.manual_seed(42)
    words = m * n // 16
    copies = cold_copies(a.copies, words * 4)
    weights = [torch.randint(-(1 << 31), 1 << 31, (words,), generator=g, dtype=torch.int64, device="cuda").to(torch.int32)
               for _ in range(copies)]
    cb = torch.randn(2 << S, generator=g, device="cuda").to(torch.float16)
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    x1 = torch.randn(n, generator=g, device="cuda").to(torch.float16)
    y1 = torch.zeros(m, dtype=torch.float16, device="cuda")
    mv = getattr(rptc_kernels, f"decompress_matvec_16_{S}_1")
    matvec_us = _graph_time_us(lambda k: mv(weights[k % copies].reshape(n // 2048, m, 128) if n % 2048 == 0 else weights[k % copies],
                                            cb, x1, y1), min(a.steps, 200))
    results = {}
    for batch in (8, 16, 32):
        x = torch.randn((batch, n), generator=g, device="cuda").to(torch.float16)
        out = torch.zeros((batch, m), dtype=torch.float16, device="cuda")
        fn = getattr(rptc_kernels, f"decompress_matmul_16_{S}_1")

        def fused(k):
            fn(weights[k % copies], cb, x, out)

        def baseline(k):
            rptc_kernels.matvec_dense(weights[k % copies], cb, W, S)
            torch.matmul(x, W.t(), out=out)

        times = {}
        for name, step in (("fused", fused), ("decode_then_gemm", baseline)):
            for k in range(10):
                step(k)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            steps = min(a.steps, 200)
            with torch.cuda.graph(graph):
                for k in range(steps):
                    step(k)
            graph.replay()
            torch.cuda.synchronize()
            evict_caches()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            times[name] = e0.elapsed_time(e1) / steps * 1e3          # us per call
        fused(0)
        rptc_kernels.matvec_dense(weights[0], cb, W, S)
        torch.cuda.synchronize()
        want = x.double() @ W.double().t()
        err = ((out.double() - want).norm() / want.norm()).item()
        flops = 2.0 * m * n * batch
        us = times["fused"]
        results[f"batch{batch}"] = {
            "us": round(us, 2), "TFLOPs": round(flops / us / 1e6, 2),
            "mfma_util": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 5),
            "hbm_GBps": round(m * n / 4 / us / 1e3, 1), "hbm_frac": round(m * n / 4 / us / 1e3 / HBM_PEAK_GBS, 4),
            "decode_then_gemm_us": round(times["decode_then_gemm"], 2),
            "speedup_vs_decode_then_gemm": round(times["decode_then_gemm"] / us, 2),
            "matvec_us": round(matvec_us, 2), "times_the_matvec": round(us / matvec_us, 2),
            "rel_l2_vs_dense": float(f"{err:.3e}"),
            "roofline": _hbm_roofline(m * n // 4, us, MEASURED_MATMUL_TRAFFIC_BYTES.get((m, n, S, batch, 2))),
        }
    other = {}
    if a.extra_shapes:
        # the other layer shapes at batch 16, fused kernel only
        del weights, W
        fn = getattr(rptc_kernels, f"decompress_matmul_16_{S}_1")
        for mm, nn in ((11008, 4096), (8192, 8192), (28672, 8192), (8192, 28672)):
            words = mm * nn // 16
            cps = cold_copies(0, words * 4)
            ws = [torch.randint(-(1 << 31), 1 << 31, (words,), generator=g, dtype=torch.int64, device="cuda").to(torch.int32)
                  for _ in range(cps)]
            x = torch.randn((16, nn), generator=g, device="cuda").to(torch.float16)
            out = torch.zeros((16, mm), dtype=torch.float16, device="cuda")
            us = _graph_time_us(lambda k: fn(ws[k % cps], cb, x, out), min(a.steps, 200))
            flops = 2.0 * mm * nn * 16
            other[f"{mm}x{nn} batch16"] = {"us": round(us, 2), "TFLOPs": round(flops / us / 1e6, 2),
                                          "mfma_util": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 5),
                                          "hbm_GBps": round(mm * nn / 4 / us / 1e3, 1),
                                          "roofline": _hbm_roofline(mm * nn // 4, us)}
            del ws
    if a.extra_shapes:
        # 3 and 4 bits per weight on the headline shape, batch 16
        for bits in (3, 4):
            mm, nn = 4096, 11008
            words = mm * nn * bits // 32
            cps = cold_copies(0, words * 4)
            ws = [torch.randint(-(1 << 31), 1 << 31, (words,), generator=g, dtype=torch.int64, device="cuda").to(torch.int32)
                  for _ in range(cps)]
            x = torch.randn((16, nn), generator=g, device="cuda").to(torch.float16)
            out = torch.zeros((16, mm), dtype=torch.float16, device="cuda")
            us = _graph_time_us(lambda k: rptc_kernels.decompress_matmul_bits(ws[k % cps], cb, x, out, bits), min(a.steps, 200))
            flops = 2.0 * mm * nn * 16
            other[f"{mm}x{nn} {bits}b batch16"] = {"us": round(us, 2), "TFLOPs": round(flops / us / 1e6, 2),
                                                  "mfma_util": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 5),
                                                  "hbm_GBps": round(mm * nn * bits / 8 / us / 1e3, 1),
                                                  "roofline": _hbm_roofline(mm * nn * bits // 8, us)}
            del ws
    line = {"metric": "fused decode+GEMM (MFMA) per call", "unit": "us", "n_gpus": 1,
            "config": {"workload": f"decompress_matmul_16_{S}_1 m={m} n={n} 2 bits/weight, {copies} rotating "
                                   f"weight copies", "launch": "graph"},
            "results": results}
    if other:
        line["other_shapes"] = other
    print(json.dumps(line))


def _graph_time_us(step, steps):
    """Average microseconds per call of step(k) over one HIP-graph replay of `steps` calls."""
    import torch
    for k in range(10):
        step(k)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for k in range(steps):
            step(k)
    graph.replay()
    torch.cuda.synchronize()
    evict_caches()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps * 1e3


def bench_other_ops(a):
    """The ops beside the headline kernel, each against the roofline that bounds it:
    decompress (writes 2mn bytes), decompress_matvec_t_16 (reads mn/4), sign_hadamard (4 bytes/element)."""
    import torch
    import rptc_kernels as rk
    rk.set_timing(False)
    g = torch.Generator(device="cuda")
    g.manual_seed(42)
    steps = min(a.steps, 200)
    res = {}

    def rand_words(k):
        return torch.randint(-(1 << 31), 1 << 31, (k,), generator=g, dtype=torch.int64, device="cuda").to(torch.int32)

    # decompress: 4096 x 4096, the reference's CPU-runnable configuration
    m, n = 4096, 4096
    comps = [rand_words(m * n // 16).reshape(m, n // 16) for _ in range(8)]
    cb16 = torch.randn(65536, generator=g, device="cuda").half()
    outs = [torch.empty((m, n), dtype=torch.float16, device="cuda") for _ in range(8)]
    us = _graph_time_us(lambda k: rk.decompress(comps[k % 8], cb16, outs[k % 8]), steps)
    byts = m * n // 4 + 2 * m * n
    # the floor of a write-bound op of this size: the framework's fill of the same output buffers
    fill_us = _graph_time_us(lambda k: outs[k % 8].fill_(1.0), steps)
    res["decompress 4096x4096"] = {"us": round(us, 2), "bytes": byts, "GBps": round(byts / us / 1e3, 1),
                                   "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4),
                                   "fill_of_the_output_us": round(fill_us, 2)}
    # transposed mat-vec, both carry modes
    for (m, n) in ((4096, 4096), (11008, 4096)):
        ncp = cold_copies(0, m * n // 4)
        streams = [rand_words(m * n // 16) for _ in range(ncp)]
        x = torch.randn(n, generator=g, device="cuda").half()
        out = torch.zeros(m, dtype=torch.float16, device="cuda")
        for mode, name in ((rk.AS_WRITTEN, "as_written"), (rk.CONTINUOUS, "continuous")):
            rk.set_carry_mode(mode)
            us = _graph_time_us(lambda k: rk.decompress_matvec_t_16(streams[k % ncp], cb16, x, out), steps)
            byts = m * n // 4
            res[f"decompress_matvec_t_16 {m}x{n} {name}"] = {
                "us": round(us, 2), "bytes": byts, "GBps": round(byts / us / 1e3, 1),
                "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)}
        rk.set_carry_mode(rk.AS_WRITTEN)
    # sign-Hadamard transform
    for (batch, n) in ((1, 4096), (1, 11008), (32, 11008), (16, 28672)):
        x = torch.randn((batch, n), generator=g, device="cuda").half()
        signs = torch.where(torch.rand(n, generator=g, device="cuda") < 0.5, -1.0, 1.0).half()
        y = torch.empty_like(x)
        us = _graph_time_us(lambda k: rk.sign_hadamard(x, signs, y), steps)
        byts = 4 * batch * n
        res[f"sign_hadamard batch {batch} n {n}"] = {"us": round(us, 2), "bytes": byts,
                                                     "GBps": round(byts / us / 1e3, 1)}
    # the general (L, S, R, V) trellis of rptc_lite.py at the reference's own setting (rptc_lite.py:141-146), 2^24
    # steps in sequences of 1024: 4 bytes of symbols read and 8 bytes of outputs written per step
    L, S, R, V, rows, T = 16, 9, 4, 2, 16384, 1024
    alphabet = torch.randn((1 << S, V), generator=g, device="cuda")
    syms = [torch.randint(0, 1 << R, (rows, T), generator=g, dtype=torch.int32, device="cuda") for _ in range(2)]
    deq = [torch.empty((rows, T, V), dtype=torch.float32, device="cuda") for _ in range(2)]
    lib = rk.library()

    def lite(k):
        rc = lib.rptc_lite_dequantize(alphabet.data_ptr(), L, S, R, V, syms[k % 2].data_ptr(), rows, T, deq[k % 2].data_ptr(),
                                      ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), None)
        assert rc == 0, rc
    us = _graph_time_us(lite, min(steps, 50))
    byts = rows * T * (4 + 4 * V)
    fill_us = _graph_time_us(lambda k: deq[k % 2].fill_(1.0), min(steps, 50))
    res[f"lite_dequantize L{L} S{S} R{R} V{V} {rows}x{T}"] = {"us": round(us, 2), "bytes": byts, "GBps": round(byts / us / 1e3, 1),
                                                            "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4),
                                                            "fill_of_the_output_us": round(fill_us, 2)}
    print(json.dumps({"metric": "other ops, microseconds per call", "unit": "us", "n_gpus": 1,
                      "config": {"launch": "graph", "steps": steps}, "results": res}))


def bench_valu_probe(a):
    """Time per instruction and SIMD of the decode's vector instructions, four waves a SIMD as in the mat-vec, against
    v_fma_f32; and from it the vector-ALU time of one 4096 x 11008 layer (12 wave-items a SIMD; per stream element
    12 v_alignbit_b32, 16 v_pk_mad_u16, 32 address ops (v_perm_b32 / v_and_or_b32), 32 v_dot2c_f32_f16)."""
    import torch
    aids = aids_library()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    names = ["v_dot2c_f32_f16", "v_pk_mad_u16", "v_perm_b32", "v_alignbit_b32", "v_and_or_b32", "v_fma_f32",
             "v_dot2c_f32_f16 on four sums in turn"]
    iters = 4000
    res = {}
    stream = torch.cuda.current_stream().cuda_stream
    for kind, name in enumerate(names):
        best = None
        for rep in range(4):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            rc = aids.rptc_probe_valu(kind, iters, cus, None, ctypes.c_void_p(stream))
            assert rc == 0, rc
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e6 / (iters * 32 * 4)          # ns per instruction and SIMD (4 waves a SIMD)
            best = t if best is None or t < best else best
        res[name] = round(best, 4)
    # the decode block by itself (registers and the LDS table only) at 1, 2 and 4 waves a SIMD
    decode = {}
    for threads in (256, 512, 1024):
        best = None
        n_el = 3000
        for rep in range(4):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            rc = aids.rptc_probe_decode(n_el, threads, cus, None, ctypes.c_void_p(stream))
            assert rc == 0, rc
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e6 / (n_el * (threads // 256))      # ns per element and SIMD
            best = t if best is None or t < best else best
        decode[f"{threads // 256} waves a SIMD"] = round(best, 2)
    # LDS read instructions, sixteen waves of a compute unit issuing them back to back
    lds = {}
    for kind, name in enumerate(["ds_read_b32", "ds_read2st64_b32", "ds_read_b64", "ds_read_b128"]):
        best = None
        n_it = 2000
        for rep in range(4):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            rc = aids.rptc_probe_lds(kind, n_it, cus, None, ctypes.c_void_p(stream))
            assert rc == 0, rc
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e6 / (n_it * 8 * 16)            # ns per instruction and compute unit (16 waves)
            best = t if best is None or t < best else best
        lds[name] = round(best, 4)
    fma = res["v_fma_f32"]
    rel = {k: round(v / fma, 3) for k, v in res.items()}
    per_element = 12 * res["v_alignbit_b32"] + 16 * res["v_pk_mad_u16"] + 16 * res["v_perm_b32"] + 16 * res["v_and_or_b32"] + 32 * res["v_dot2c_f32_f16"]
    print(json.dumps({"metric": "vector instruction issue time, ns per instruction and SIMD", "unit": "ns", "n_gpus": 1,
                      "config": {"waves_per_simd": 4, "instructions_per_wave": iters * 32}, "results": res,
                      "relative_to_v_fma_f32": rel, "lds_read_ns_per_instruction_and_cu": lds,
                      "decode_block_ns_per_element_and_simd": decode,
                      "decode_block_us_per_4096x11008_layer": round(12 * decode["4 waves a SIMD"] / 1e3, 3),
                      "decode_valu_us_per_4096x11008_layer": round(12 * per_element / 1e3, 3)}))


def bench_quantize(a):
    """The Viterbi search kernel (the quantizer's inner loop) on the rows of one 4096 x 4096 layer:
    trellis state updates per second against the vector-ALU rate that bounds it, with the same search in
    framework ops on the GPU and the C restatement on the host's cores beside it."""
    import time
    import numpy as np
    import torch
    import rptc_kernels as rk
    from rptc_kernels import quantize
    g = torch.Generator(device="cuda")
    g.manual_seed(42)
    cb = torch.randn(512, generator=g, device="cuda").half()
    rows, steps = 512, 2048                                         # two rows per CU, n = 4096
    tg = torch.randn((rows, steps, 2), generator=g, device="cuda") * 0.7
    best = None
    for _ in range(max(2, min(a.steps, 5))):
        sym, cost, end, ms = rk.viterbi_pairs(tg, cb)
        best = ms if best is None else min(best, ms)
    updates = rows * steps * 65536
    # vector-ALU ceiling: 256 CUs x 64 lanes x 2.4 GHz lane-ops/s; a state update costs 5 vector ops
    # (byte permute, add, and compare + two selects in the minimum over predecessors)
    valu_peak = 256 * 64 * 2.4e9
    res = {"viterbi_pairs rows 512 steps 2048": {
        "ms": round(best, 3), "state_updates_per_s": float(f"{updates / best * 1e3:.4e}"),
        "us_per_step_per_row_round": round(best * 1e3 / steps / (rows / 256), 3),
        "vector_ops_per_update": 5, "frac_of_valu_peak": round(updates * 5 / (best * 1e-3) / valu_peak, 4)}}
    # 3 and 4 bits per weight: 6 and 8 stream bits per step, 64 and 256 predecessors per state
    for bits in (3, 4):
        b_ms = None
        for _ in range(3):
            _, _, _, ms = rk.viterbi_pairs(tg[:256], cb, bits=bits)
            b_ms = ms if b_ms is None else min(b_ms, ms)
        res[f"viterbi_pairs {bits} bits rows 256 steps 2048"] = {
            "ms": round(b_ms, 3), "state_updates_per_s": float(f"{256 * steps * 65536 / b_ms * 1e3:.4e}")}
    # the reference's own trellis (2 bits and one alphabet value per step): 6 vector ops per update
    # (mixed-precision subtract, square, add, and the minimum over four predecessors)
    ab = torch.randn(1 << 16, generator=g, device="cuda").half()
    tgs = torch.randn((256, 4096), generator=g, device="cuda")
    best_s = None
    for _ in range(3):
        _, cost_s, _, ms = rk.viterbi_scalar(tgs, ab)
        best_s = ms if best_s is None else min(best_s, ms)
    res["viterbi_scalar L=16 rows 256 steps 4096"] = {
        "ms": round(best_s, 3), "state_updates_per_s": float(f"{256 * 4096 * 65536 / best_s * 1e3:.4e}"),
        "us_per_step": round(best_s * 1e3 / 4096, 3), "mse_unit_gaussian_2_bits": round(float(cost_s.sum()) / (256 * 4096), 4)}
    # the same search in framework ops on the GPU (64 rows, 256 steps)
    table = quantize.decode_table(cb, 8)
    small = tg[:64, :256].contiguous()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    sym_t, cost_t = quantize.viterbi_pairs(small, table)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    sym_h, cost_h, _, _ = rk.viterbi_pairs(small, cb)
    res["framework ops rows 64 steps 256"] = {"ms": round(dt * 1e3, 2),
                                              "state_updates_per_s": float(f"{64 * 256 * 65536 / dt:.4e}"),
                                              "same_path_as_kernel": bool(torch.equal(sym_t, sym_h.long()))}
    if not a.no_cpu:
        from oracle import rptc_oracle
        t_np, c_np = table.cpu().numpy(), small[0, :64].cpu().numpy()
        t0 = time.perf_counter()
        osym, ocost, _ = rptc_oracle.viterbi(t_np, 4, c_np)
        dt = time.perf_counter() - t0
        res["cpu oracle 1 row 64 steps (1 core)"] = {"ms": round(dt * 1e3, 2),
                                                     "state_updates_per_s": float(f"{64 * 65536 / dt:.4e}"),
                                                     }
        sym_1, _, _, _ = rk.viterbi_pairs(small[:1, :64].contiguous(), cb)
        res["cpu oracle 1 row 64 steps (1 core)"]["same_path_as_kernel"] = bool(np.array_equal(osym, sym_1[0].cpu().numpy()))
    # a whole layer through quantize_matrix (search + copies to the host)
    W = torch.randn((4096, 4096), generator=g, device="cuda") * 0.7
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    _, mse = quantize.quantize_matrix(W, cb, 8)
    torch.cuda.synchronize()
    res["quantize_matrix 4096x4096"] = {"s": round(time.perf_counter() - t0, 3), "mse_over_variance": round(mse / float(W.var()), 4)}
    print(json.dumps({"metric": "Viterbi search, trellis state updates per second", "unit": "updates/s", "n_gpus": 1,
                      "value": res["viterbi_pairs rows 512 steps 2048"]["state_updates_per_s"], "data": "synthetic",
                      "config": {"workload": "65536-state trellis, 4 bits and two weights per step, Gaussian targets, S=8"},
                      "results": res}))


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    if a.valu_probe:
        bench_valu_probe(a)
        return
    if a.matmul:
        bench_matmul(a)
        return
    if a.other_ops:
        bench_other_ops(a)
        return
    if a.quantize:
        bench_quantize(a)
        return
    if a.decode:
        from rptc_kernels.llama_decode import LlamaShape, QuantizedLlama, greedy_decode
        shape = LlamaShape(layers=a.decode_layers)
        t0 = time.perf_counter()
        model = QuantizedLlama(shape, S=a.S, quantize_init=a.decode_quantized)
        torch.cuda.synchronize()
        build_s = time.perf_counter() - t0
        g = torch.Generator().manual_seed(42)
        prompt = torch.randint(0, shape.vocab, (512,), generator=g)
        res = {}
        if a.decode_quantized:
            blk = model.blocks[0]
            res["quantizer"] = {"seconds_for_the_model": round(build_s, 1),
                                "mse_of_the_normalised_weights_layer_0": {
                                    name: round(getattr(blk, name).quantization_mse, 4)
                                    for name in ("qkv_proj", "o_proj", "gate_up_proj", "down_proj")}}
        for mode in (("fused_graph", "glue_graph") if a.decode_quantized else
                     ("fused_graph", "fused", "glue_graph", "torch_graph", "torch")):
            model.k_cache.zero_()
            model.v_cache.zero_()
            toks, dt = greedy_decode(model, prompt, 128, mode=mode)
            res[mode] = {"tok_per_s": round(127 / dt, 1), "ms_per_token": round(dt / 127 * 1e3, 3)}
        stream_bytes = sum(b.compressed_bytes() for blk in model.blocks for b in blk.children())
        print(json.dumps({"metric": "decode tok/s Llama-2-7B-shape bs=1", "value": res["fused_graph"]["tok_per_s"], "unit": "tok/s",
                          "n_gpus": 1, "data": "synthetic",
                          "config": {"workload": f"{shape.layers} layers d=4096 heads=32 mlp=11008 vocab=32000, random-init, "
                                                 + ("projections random-init dense weights quantized to 2 bits (factorisation + trellis search), "
                                                    "their scales and biases applied in the kernels " if a.decode_quantized else
                                                    "projections as seeded random 2-bit streams ") +
                                                 f"({stream_bytes} bytes), prompt 512 "
                                                 f"random ids, 128 greedy tokens; fused_graph = five launches per layer (element-wise steps inside the projections) in one HIP graph per token; glue_graph = nine launches per layer"},
                          "results": res}))
        return
    a.copies = cold_copies(a.copies, a.m * a.n // 4)
    runner = Runner(a.m, a.n, a.S, a.copies)
    if a.pmc_probe:
        # calibration: an int32 -> float32 conversion copy is a plain streaming kernel that reads
        # 64 MiB and writes 64 MiB
        import rptc_kernels as rk
        src = torch.randint(0, 1 << 20, (16 << 20,), dtype=torch.int32, device="cuda")
        dst = torch.empty(16 << 20, dtype=torch.float32, device="cuda")
        stream = torch.cuda.current_stream().cuda_stream
        for k in range(8):
            dst.copy_(src)
            runner.launch(k, stream)
        torch.cuda.synchronize()
        # the chain: one launch of `copies` independent layers, twice (counters per dispatch = per `copies` layers)
        outs = torch.zeros((a.copies, a.m), dtype=torch.float16, device="cuda")
        chain = rk.MatvecChain([(runner.weights[k], runner.x, outs[k]) for k in range(a.copies)], runner.codebook)
        for _ in range(2):
            chain.run(carry_mode=0, timed=False)
        torch.cuda.synchronize()
        # the transposed mat-vec (4096 x 4096, scalar 2^16 codebook, both carry modes) and the batched product (batch 16)
        g = torch.Generator(device="cuda")
        g.manual_seed(7)
        rk.set_timing(False)
        cb16 = torch.randn(65536, generator=g, device="cuda").half()
        xt = torch.randn(4096, generator=g, device="cuda").half()
        yt = torch.zeros(4096, dtype=torch.float16, device="cuda")
        streams = [torch.randint(-(1 << 31), 1 << 31, (4096 * 4096 // 16,), generator=g, dtype=torch.int64, device="cuda").to(torch.int32)
                   for _ in range(8)]
        for mode in (rk.AS_WRITTEN, rk.CONTINUOUS):
            rk.set_carry_mode(mode)
            for k in range(8):
                rk.decompress_matvec_t_16(streams[k], cb16, xt, yt)
        rk.set_carry_mode(rk.AS_WRITTEN)
        xb = torch.randn((16, a.n), generator=g, device="cuda").half()
        yb = torch.zeros((16, a.m), dtype=torch.float16, device="cuda")
        for k in range(8):
            getattr(rk, f"decompress_matmul_16_{a.S}_1")(runner.weights[k % a.copies], runner.codebook, xb, yb)
        torch.cuda.synchronize()
        print(f"pmc-probe: 8 conversion copies of {src.numel() * 4} bytes in / {dst.numel() * 4} bytes out, "
              f"8 launches of {runner.bytes} compressed bytes, 2 chain launches of {a.copies} such layers, "
              f"8 + 8 launches of decompress_matvec_t_16 on 4096 x 4096 (as written, continuous), "
              f"8 launches of the batch-16 product on {a.m} x {a.n}")
        return
    err = runner.check()
    per_launch = None
    if a.launch == "chain":
        # the per-launch pattern first (one launch per step in a HIP graph), then the chain, which is the figure reported
        _, g_ms = runner.run(a.steps, a.warmup, "graph")
        per_launch = {"launch": "graph", "launch_us": round(g_ms / a.steps * 1e3, 3),
                      "GBps": round(runner.bytes / (g_ms / a.steps * 1e-3) / 1e9, 2),
                      "frac": round(runner.bytes / (g_ms / a.steps * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        wall, ev_ms, err_chain = runner.chain_run(a.steps, a.warmup)
    else:
        wall, ev_ms = runner.run(a.steps, a.warmup, a.launch)
    ms_per_step = wall * 1e3 / a.steps
    launch_ms = ev_ms / a.steps
    value = runner.bytes / (ms_per_step * 1e-3) / 1e9
    achieved = runner.bytes / (launch_ms * 1e-3) / 1e9
    line = {
        "metric": "fused decode+GEMV GB/s (compressed)",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": f"decompress_matvec_16_{a.S}_1 m={a.m} n={a.n} 2 bits/weight batch 1 "
                        f"(Llama-2-7B down_proj shape), {a.copies} rotating weight copies of {runner.bytes} bytes "
                        f"({a.copies * runner.bytes >> 20} MiB), caches flushed before the timed region",
            "distinct_copies_touched": min(a.steps, a.copies),
            "launch": a.launch if a.launch != "chain" else "chain: the steps are the layers of one rptc_decompress_matvec_chain launch "
                                                            "(independent layers, an output buffer per layer)",
            "accumulate": "f32",
            "carry_mode": "as_written",
            "compressed_bytes": runner.bytes,
            "rel_l2_vs_dense": float(f"{err:.3e}"),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": None,
            "launch_us": round(launch_ms * 1e3, 3),
        },
    }
    kernel = "matvec_steady_kernel" if a.launch == "chain" else "matvec_kernel"
    line["roofline"]["traffic"], line["roofline"]["traffic_measured_at"] = measured_traffic(kernel, a.m, a.n)
    if per_launch is not None:
        line["roofline"]["kernel"] = ("matvec_steady_kernel (the form rptc_decompress_matvec_chain takes for independent layers of one shape): "
                                      "achieved = steps x compressed bytes / the one launch's duration; launch_us is per layer")
        per_launch["traffic"], per_launch["traffic_measured_at"] = measured_traffic("matvec_kernel", a.m, a.n)
        line["per_launch"] = per_launch
    # the floor of this workload on this machine, in the same launch pattern (graph replay over the
    # same rotating buffers): an empty launch, and a kernel that only reads the stream
    aids = aids_library()
    grid = -(-a.m // (2 * -(-a.m // (2 * torch.cuda.get_device_properties(0).multi_processor_count))))

    def floor_us(call):
        steps = min(a.steps, 400)
        for k in range(10):
            call(k, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            cs = torch.cuda.current_stream().cuda_stream
            for k in range(steps):
                call(k, cs)
        graph.replay()
        torch.cuda.synchronize()
        evict_caches()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps * 1e3

    def call_empty(k, cs):
        if aids.rptc_probe_empty(grid, ctypes.c_void_p(cs)):
            raise RuntimeError("rptc_probe_empty failed")

    def call_read(k, cs):
        w = runner.weights[k % len(runner.weights)]
        if aids.rptc_probe_read(w.data_ptr(), runner.bytes, None, ctypes.c_void_p(cs)):
            raise RuntimeError("rptc_probe_read failed")

    def chain_read_us():
        """The chain's pattern with nothing decoded: one persistent launch that reads every layer's stream."""
        cus = torch.cuda.get_device_properties(0).multi_processor_count
        if runner.bytes % (16 * cus):
            return None
        ptrs = torch.tensor([w.data_ptr() for w in runner.weights], dtype=torch.int64, device="cuda")
        cs = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        best = None
        for rep in range(3):
            evict_caches()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            rc = aids.rptc_probe_read_chain(ptrs.data_ptr(), len(runner.weights), a.steps, runner.bytes, cus, None, cs)
            e1.record()
            torch.cuda.synchronize()
            if rc:
                return None
            us = e0.elapsed_time(e1) / a.steps * 1e3
            best = us if rep > 0 and (best is None or us < best) else best
        return best

    if a.launch in ("graph", "chain"):
        empty_us, read_us = floor_us(call_empty), floor_us(call_read)
        line["roofline"]["floor"] = {
            "empty_launch_us": round(empty_us, 3),
            "read_only_us": round(read_us, 3),
            "read_only_GBps": round(runner.bytes / read_us / 1e3, 1),
            "note": "same bytes, same graph-replayed launch pattern: an empty kernel, and a kernel that only reads the stream",
        }
        if a.launch == "chain":
            try:
                cr = chain_read_us()
            except Exception as e:      # an optional figure: the line is printed without it
                print(f"bench.py: the persistent read-only probe failed: {e}", file=sys.stderr)
                cr = None
            if cr is not None:
                line["roofline"]["floor"]["chain_read_only_us"] = round(cr, 3)
                line["roofline"]["floor"]["chain_read_only_GBps"] = round(runner.bytes / cr / 1e3, 1)
                line["roofline"]["floor"]["chain_note"] = ("one persistent launch, one workgroup per compute unit, that only reads the same layers "
                                                           "(a layer ahead, 1 KiB per wave request): the memory floor of the chain's pattern")
    if a.extra_shapes:
        extra = {}
        for (m, n) in ((4096, 4096), (11008, 4096), (8192, 8192), (28672, 8192), (8192, 28672)):
            r = Runner(m, n, a.S, cold_copies(0, m * n // 4))
            r.check()
            _, ms = r.run(a.steps, a.warmup, a.launch)
            us = ms / a.steps * 1e3
            extra[f"{m}x{n}"] = {"launch_us": round(us, 3), "GBps": round(r.bytes / us / 1e3, 1),
                                 "frac": round(r.bytes / us / 1e3 / HBM_PEAK_GBS, 4)}
            del r
            torch.cuda.empty_cache()
        for bits in (3, 4):
            for (m, n) in ((4096, 11008), (11008, 4096)):
                r = Runner(m, n, a.S, cold_copies(0, m * n * bits // 8), bits=bits)
                r.check()
                _, ms = r.run(a.steps, a.warmup, a.launch)
                us = ms / a.steps * 1e3
                extra[f"{m}x{n} {bits}b"] = {"launch_us": round(us, 3), "GBps": round(r.bytes / us / 1e3, 1),
                                            "frac": round(r.bytes / us / 1e3 / HBM_PEAK_GBS, 4)}
                del r
                torch.cuda.empty_cache()
        line["other_shapes"] = extra
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(runner)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
