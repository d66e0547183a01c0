#!/usr/bin/env python3
"""Benchmark of the Linear4bit forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one pass of the hot path over one batch of synthetic input, everything
resident in HBM: per-token symmetric int4 quantization of the fp16 activations, the
int4 x int4 GEMM and the fused fp16 dequant epilogue (``Sequential(SymQuantizer,
Linear4bitSQ)``).  The GEMM runs on the matrix path for 6-bit floats (every int4 value is
exactly an E3M2 number and the float32 accumulation of their products is exact, so the result
is the integer GEMM bit for bit at twice the i8 MFMA rate); the same step on the i8 MFMA
kernels is timed beside it (``integer_path``).  The workload is the prefill configuration
the metric is quoted on: M = 2048 tokens, K = N = 4096 (a Llama-2-7B attention
projection), activations ~N(0,1) with 1 % heavy-tailed channels, weights uniform random
nibbles with per-channel scales.

Prints ONE JSON line.  ``value`` is 2*M*N*K / (time per step) in TOPS for the whole step timed as eager module
calls (how the reference's harness times a layer, test/benchmark.py:24-39); the same K steps as one HIP graph
replayed once are reported beside it (``graph_ms_per_step``).
``roofline`` describes the dominant kernel (the fused GEMM): achieved = 2*M*N*K / its own
average duration, measured with HIP events around max(steps, 1000) back-to-back launches on the
launch stream (so the figure does not depend on ``--steps``), against the published dense peak
of the matrix instruction it uses; ``traffic`` is read from the rocprofv3 summary under
``profiles/``.  ``decode`` times configuration 2 as it is stated (binary16 activations in,
quantized per token, GEMM, dequant: the single entry point ``quantize_linear4bit_forward``) with
its algorithmic bytes 2MK + NK/2 + 2N + 2MN, beside the GEMM alone on pre-quantized activations
and a read-only kernel over the same weight bytes (the floor of a launch of that size);
``roofline_decode`` is the WORST of the Llama-2-7B rows.  ``quantizer`` reports the quantizer
against HBM, ``harness`` reproduces the reference's own benchmark table (module-level eager wall time of the 4-bit
layers and of the fp16 torch.nn.Linear at its six layer sizes), ``fanout`` one quantizer feeding several
projections, ``cpu_baseline`` the CPU fake-quant path on the host.

Every timed loop is preceded by PREWARM_STEPS untimed steps on top of ``--warmup`` (after an idle
period the part needs about a millisecond of work to reach the clock it then holds).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, published
PREWARM_STEPS = 300       # untimed steps before the W warm-up steps of every timed loop (about 10 ms of GPU work)
PEAK_FP6_TOPS = 10100.0   # MI355X dense fp6 / fp4 MFMA, published
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, published
EVENT_TIMED_LAUNCHES = 1000  # at least this many back-to-back launches behind every per-kernel figure


def profile_traffic_bytes(name, kernel):
    """HBM bytes per launch (fetched + written) of `kernel` from the rocprofv3 --pmc summary profiles/<name>:
    the line 'dispatches N  fetch avg F KiB (max ..)  write avg W KiB (max ..)' after the kernel's name under
    'HBM traffic per launch'.  None when the summary is not there."""
    import re

    try:
        text = open(os.path.join(ROOT, "profiles", name)).read()
    except OSError:
        return None
    at = text.find("HBM traffic per launch")
    at = text.find(kernel, at) if at >= 0 else -1
    m = re.search(r"fetch avg (\d+) KiB.*?write avg (\d+) KiB", text[at:]) if at >= 0 else None
    return (int(m.group(1)) + int(m.group(2))) * 1024 if m else None


def profile_shape_traffic_bytes(name, kernel, workgroups):
    """HBM bytes per launch (fetched + written) of `kernel` at the launch shape with `workgroups` workgroups, from the
    per-shape lines 'workgroups W x T threads: ... fetch avg F KiB  write avg W KiB' of profiles/<name>."""
    import re

    try:
        text = open(os.path.join(ROOT, "profiles", name)).read()
    except OSError:
        return None
    for m in re.finditer(r"^  (\S.*)\n    workgroups (\d+) x \d+ threads:.*?fetch avg (\d+) KiB\s+write avg (\d+) KiB", text, re.M):
        if kernel in m.group(1) and int(m.group(2)) == workgroups:
            return (int(m.group(3)) + int(m.group(4))) * 1024
    return None


def heavy_tail_acts(M, K, seed, frac=0.01):
    import torch

    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    n = max(1, round(frac * K))
    ch = torch.randperm(K, generator=g)[:n]
    z = torch.randn(M, n, generator=g)
    chi = (torch.randn(M, n, 3, generator=g) ** 2).sum(-1) / 3.0
    x[:, ch] = z / chi.sqrt()  # Student-t, 3 degrees of freedom
    return x.to(torch.float16)


def random_weights(N, K, seed, dev):
    import torch

    g = torch.Generator().manual_seed(seed)
    packed = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)  # uniform nibbles in [-8, 7]
    scales = (torch.rand(N, 1, generator=g) * 0.009 + 0.001).to(torch.float16)
    return packed.to(dev), scales.to(dev)


def event_time_us(fn, n, warm):
    """Average GPU time of fn() over n back-to-back launches, HIP events on the current stream."""
    import torch

    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(n):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / n


def graph_time_us(fns, reps=5):
    """Kernels too short to be launched back-to-back from Python (a few microseconds) are
    recorded once into a HIP graph and replayed: microseconds per call, best of reps."""
    import torch

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for f in fns[:2]:
            f()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for f in fns:
            f()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    graph.replay()
    e1.record()
    torch.cuda.synchronize()
    # replay for about 3 ms before timing: after an idle period the part needs about a millisecond of work to reach
    # the clock it then holds (a 200-step run of the 30 us step measures 10 % slower than a 2000-step one)
    for _ in range(min(400, max(1, int(3.0 / max(e0.elapsed_time(e1), 1e-3))))):
        graph.replay()
    torch.cuda.synchronize()
    best = None
    for _ in range(reps):
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e3 / len(fns)
        best = t if best is None else min(best, t)
    return best


def eager_wall_us(modules, x, steps=1000, warm=200, reps=3):
    """Wall time per eager call of modules[i % n](x): perf_counter around a loop that ends in synchronize(); the
    best of `reps` such loops (a host-bound figure of a few microseconds picks up every hiccup of the host)."""
    import torch

    n = len(modules)
    for i in range(warm):
        modules[i % n](x)
    torch.cuda.synchronize()
    best = None
    for _ in range(reps):
        t0 = time.perf_counter()
        for i in range(steps):
            modules[i % n](x)
        torch.cuda.synchronize()
        t = (time.perf_counter() - t0) * 1e6 / steps
        best = t if best is None else min(best, t)
    return best


def shader_clock_mhz():
    """The shader clock the driver reports right now (the level marked '*' in pp_dpm_sclk of the first GPU), or
    None where that file is not readable."""
    import glob
    import re

    for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
        try:
            text = open(path).read()
        except OSError:
            continue
        m = re.search(r"(\d+)\s*Mhz\s*\*", text, re.I)
        if m:
            return int(m.group(1))
    return None


class ClockSampler:
    """Samples shader_clock_mhz() from a thread while a timed loop runs: the clock the part held under that load."""

    def __init__(self, period_s=0.002):
        import threading

        self.period, self.samples, self._stop = period_s, [], threading.Event()
        self._t = threading.Thread(target=self._run, daemon=True)

    def _run(self):
        while not self._stop.is_set():
            v = shader_clock_mhz()
            if v is None:
                return
            self.samples.append(v)
            time.sleep(self.period)

    def __enter__(self):
        self._t.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._t.join(timeout=1.0)

    def summary(self):
        if not self.samples:
            return None
        s = sorted(self.samples)
        return {"median_mhz": s[len(s) // 2], "min_mhz": s[0], "max_mhz": s[-1], "samples": len(s)}


def harness_section(dev, quick=False):
    """The reference's own benchmark (test/benchmark.py:8-39, 54-100) on this GPU: x = rand(1, seq_len, in) as
    binary16, weights integers in [-8, 7) with unit scales, module-level eager wall time in ms (5 warm-up + 100 calls
    per run, mean of `runs` runs) of Sequential(SymQuantizer, Linear4bitSQ), Sequential(SymQuantizer,
    Linear4bitDUSQ) and the fp16 torch.nn.Linear they replace, at its six layer sizes, for seq_len 2048 (its
    default), 16 and 1; plus the 4-bit layer on the 6-bit float matrix path at seq_len 2048 (enable_fp6, not in the
    reference)."""
    import torch

    from duqlinear4bitcuda_amd.nn import Linear4bitDUSQ, Linear4bitSQ, SymQuantizer

    sizes = [(4096, 4096), (5120, 5120), (8192, 8192), (4096, 11008), (5120, 13824), (8192, 28672)]
    if quick:
        sizes = sizes[:1]
    runs = 3

    def module_benchmark(module, x):
        for _ in range(5):
            module(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(100):
            module(x)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1000 / 100

    def mean_ms(module, x):
        module_benchmark(module, x)   # one untimed run: clock ramp, lazy set-up
        return sum(module_benchmark(module, x) for _ in range(runs)) / runs

    out = []
    for (fin, fout) in sizes:
        base = torch.nn.Linear(fin, fout, bias=False).to(dev).half()
        base.weight.data = torch.randint_like(base.weight.data, low=-8, high=7).half()
        s_w = torch.ones((fout, 1), dtype=torch.float16, device=dev)
        with torch.no_grad():
            sq = Linear4bitSQ.from_float(base, weight_scales=s_w).to(dev)
            du = Linear4bitDUSQ.from_float(base, weight_scales_1=s_w, weight_scales_2=s_w.clone()).to(dev)
            int4 = torch.nn.Sequential(SymQuantizer(input_clip_ratio=1.0), sq)
            int4duq = torch.nn.Sequential(SymQuantizer(input_clip_ratio=1.0), du)
            row = {"in": fin, "out": fout}
            for seq in (2048, 16, 1):
                x = torch.rand((1, seq, fin), device=dev).half()
                t4, td, tf = mean_ms(int4, x), mean_ms(int4duq, x), mean_ms(base, x)
                r = {"int4_ms": round(t4, 4), "int4_duq_ms": round(td, 4), "fp16_ms": round(tf, 4),
                     "speedup_int4": round(tf / t4, 3), "speedup_int4_duq": round(tf / td, 3)}
                if seq == 2048 and fin % 128 == 0 and fout % 16 == 0:
                    sq.enable_fp6()
                    fp6 = torch.nn.Sequential(SymQuantizer(1.0, shadow="only", shadow_min_rows=1), sq)
                    t6 = mean_ms(fp6, x)
                    r.update({"int4_fp6_path_ms": round(t6, 4), "speedup_int4_fp6_path": round(tf / t6, 3)})
                    del sq._buffers["weight_shadow"]
                row[f"seq{seq}"] = r
        out.append(row)
        del base, sq, du, int4, int4duq
    return {"what": "module-level eager wall time as test/benchmark.py of the reference measures it (bsz 1; 5 + 100 calls, "
                    f"mean of {runs} runs after one untimed run), fp16 = torch.nn.Linear (hipBLASLt) on the same GPU",
            "rows": out}


def fanout_section(dev):
    """One quantized activation feeding several projections of a Llama-2-7B block as ONE GEMM over the concatenated
    weight (q/k/v: N = 3 x 4096; gate/up: N = 2 x 11008), M = 2048: the quantizer's share of the step shrinks with
    the width it feeds.  HIP-graph timed module steps, 6-bit float path and integer path."""
    import torch

    from duqlinear4bitcuda_amd.nn import Linear4bitSQ, SymQuantizer

    out = []
    M, K = 2048, 4096
    x = heavy_tail_acts(M, K, seed=8).to(dev)
    for name, N in (("one projection", 4096), ("q/k/v as one GEMM", 3 * 4096), ("gate/up as one GEMM", 2 * 11008)):
        w, sw = random_weights(N, K, seed=88, dev=dev)
        lin = Linear4bitSQ(K, N, bias=False).to(dev)
        lin.weight.copy_(w)
        lin.weight_scales = sw
        q_i8 = SymQuantizer(1.0)
        q_f6 = SymQuantizer(1.0, shadow="only", shadow_min_rows=1)
        us_i8 = graph_time_us([lambda: lin(q_i8(x))] * 6)
        lin.enable_fp6()
        us_f6 = graph_time_us([lambda: lin(q_f6(x))] * 6)
        pq = q_f6(x)
        us_gemm = graph_time_us([lambda: lin(pq)] * 6)
        ops = 2.0 * M * N * K
        out.append({"what": name, "M": M, "K": K, "N": N, "fp6_step_us": round(us_f6, 1), "fp6_TOPS": round(ops / us_f6 / 1e6, 1),
                    "fp6_gemm_only_us": round(us_gemm, 1), "quantizer_share": round(1.0 - us_gemm / us_f6, 3),
                    "integer_step_us": round(us_i8, 1), "integer_TOPS": round(ops / us_i8 / 1e6, 1)})
        del lin, w
    return out


LLAMA7B_DECODE = [(M, N, 4096) for N in (4096, 11008) for M in (1, 4, 16)]   # configuration 2


def decode_section(dev, quick, eager=True):
    """HBM-bound decode at configuration 2 and around it.  Per shape, HIP-graph timed, with the weights rotated
    over more than 512 MB of distinct buffers so that no launch finds its weights in a cache:
      us            binary16 activations in -> per-token quantize -> GEMM -> fp16 out, the single entry point
                    (one launch up to eight rows and for nine to sixteen short ones, quantizer + GEMM launches above)
      gemm_only_us  the GEMM + dequant launch alone on pre-quantized activations
      read_floor_us a kernel that only reads the same N*K/2 weight bytes with the decode access pattern
      module_graph_us  the same step through the drop-in modules, Sequential(SymQuantizer, Linear4bitSQ) on an input
                    [1, M, K] (test/benchmark.py:54-70 of the reference), replayed from a HIP graph
      module_eager_us  the same modules called eagerly: wall time per call (time.perf_counter around a loop that
                    ends in synchronize(), as test/benchmark.py:24-39), which is what a caller without graphs gets:
                    host time per call when that exceeds the kernels' time
      module_launches  library calls per module step
    GBps / frac_hbm use `us` and the algorithmic bytes 2MK + NK/2 + 2N + 2MN."""
    import torch

    from duqlinear4bitcuda_amd import _HIP as hip
    from duqlinear4bitcuda_amd.nn import Linear4bitSQ, SymQuantizer

    out = []
    shapes = list(LLAMA7B_DECODE)
    if not quick:
        shapes += [(8, 4096, 4096), (32, 4096, 4096), (64, 11008, 4096), (1, 4096, 11008), (16, 4096, 11008), (1, 28672, 8192),
                   (1, 8192, 28672), (16, 28672, 8192),
                   # sixteen rows of 2048 elements: one launch (the MFMA decode kernel quantizes the rows itself)
                   (16, 2048, 2048), (16, 8192, 2048)]
    for (M, N, K) in shapes:
        wbytes = N * K // 2
        nbuf = min(96, max(3, int(600e6 // wbytes) + 1))
        ws = [torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, device=dev) for _ in range(nbuf)]
        x = torch.randn(M, K, device=dev).half()
        xq, sx = hip.quantize_rows_sym(x)
        sw = (torch.rand(N, 1, device=dev) * 0.009 + 0.001).half()
        us = graph_time_us([(lambda w=w: hip.quantize_linear4bit_forward(x, w, sw)) for w in ws] * 2)
        us_gemm = graph_time_us([(lambda w=w: hip.linear4bit_forward(hip.EPI_SYM, xq, sx, None, w, sw)) for w in ws] * 2)
        us_read = graph_time_us([(lambda w=w: hip.probe_read(w)) for w in ws] * 2)
        # the drop-in modules, one layer per weight buffer (the same rotation)
        x3 = x.view(1, M, K)
        models = []
        for w in ws:
            layer = Linear4bitSQ(K, N, bias=False).to(dev)
            layer.weight = w
            layer.weight_scales = sw
            models.append(torch.nn.Sequential(SymQuantizer(1.0), layer))
        us_mod_graph = graph_time_us([(lambda m=m: m(x3)) for m in models] * 2)
        us_mod_eager = eager_wall_us(models, x3) if eager else float("nan")
        byts = 2 * M * K + wbytes + 2 * N + 2 * M * N
        out.append({"M": M, "N": N, "K": K, "us": round(us, 3), "GBps": round(byts / us / 1e3, 1),
                    "frac_hbm": round(byts / us / 1e3 / PEAK_HBM_GBS, 4),
                    "launches": 1 if hip.quantize_linear4bit_one_launch(M, N, K) else 2,
                    "module_graph_us": round(us_mod_graph, 3), "module_eager_us": round(us_mod_eager, 3) if eager else None,
                    "module_launches": 1 if hip.quantize_linear4bit_one_launch(M, N, K) else 2,
                    "module_library_calls": 1 if M <= 1024 else 2,
                    "gemm_only_us": round(us_gemm, 3),
                    "gemm_only_GBps": round((byts - 2 * M * K + M * K // 2 + 2 * M) / us_gemm / 1e3, 1),
                    "read_floor_us": round(us_read, 3), "read_floor_GBps": round(wbytes / us_read / 1e3, 1),
                    "frac_of_read_floor": round(us_read / us, 4), "gemm_kernel_family": hip.gemm_kernel_for(M, N, K),
                    "weight_buffers": nbuf})
        del ws, models
    return out


def quantizer_section(dev):
    import torch

    from duqlinear4bitcuda_amd import _HIP as hip

    out = []
    for (M, K) in [(2048, 4096), (2048, 11008)]:
        nbuf = min(64, max(3, int(600e6 // (M * K * 2)) + 1))
        xs = [torch.randn(M, K, device=dev).half() for _ in range(nbuf)]
        us = graph_time_us([(lambda x=x: hip.quantize_rows_sym(x)) for x in xs] * 2)
        byts = 2 * M * K + M * K // 2 + 2 * M
        out.append({"M": M, "K": K, "out": "int4", "us": round(us, 3), "GBps": round(byts / us / 1e3, 1),
                    "frac_hbm": round(byts / us / 1e3 / PEAK_HBM_GBS, 4)})
        us = graph_time_us([(lambda x=x: hip.quantize_rows_sym_bf6(x, with_q=False)) for x in xs] * 2)
        byts = 2 * M * K + M * K * 3 // 4 + 2 * M
        out.append({"M": M, "K": K, "out": "e3m2 shadow", "us": round(us, 3), "GBps": round(byts / us / 1e3, 1),
                    "frac_hbm": round(byts / us / 1e3 / PEAK_HBM_GBS, 4)})
        del xs
    return out


def asym_section(dev):
    """Dual-uniform / asymmetric configuration (M=512, K=N=4096, activations ~U[0,6]): one module step
    (quantize + GEMM + dequant, two launches) in the reference-faithful mode and in the row-sum mode."""
    import torch

    from duqlinear4bitcuda_amd.nn import Linear4bitASQ, Linear4bitASQRowSum, LinearQuant4bitDUASQ, LinearQuant4bitDUASQRowSum

    M, K, N = 512, 4096, 4096
    g = torch.Generator().manual_seed(4)
    x = (torch.rand(M, K, generator=g) * 6).half().to(dev)
    lin = torch.nn.Linear(K, N, bias=False).half()
    with torch.no_grad():
        lin.weight.copy_((torch.randn(N, K, generator=g) * 0.02).half())
    ref_mode = Linear4bitASQ.from_linear(lin).to(dev)
    rowsum_mode = Linear4bitASQRowSum.from_linear(lin.to(dev))
    true = x.float() @ lin.weight.detach().float().t()
    out = {"M": M, "N": N, "K": K}
    for name, mod in (("reference_mode", ref_mode), ("rowsum_mode", rowsum_mode)):
        us = graph_time_us([lambda: mod(x)] * 20)
        y = mod(x).float()
        out[name] = {"step_us": round(us, 2), "TOPS": round(2.0 * M * N * K / us / 1e6, 1),
                     "rel_error_vs_fp32_matmul": round(float((y.detach() - true).norm() / true.norm()), 4)}
        # the same layer on the 6-bit float matrix path (64-row tiles at this size): same bits
        y_int = mod(x)
        mod.enable_fp6()
        same = bool(torch.equal(mod(x).view(torch.int16), y_int.view(torch.int16)))
        us6 = graph_time_us([lambda: mod(x)] * 20)
        out[name].update({"fp6_step_us": round(us6, 2), "fp6_TOPS": round(2.0 * M * N * K / us6 / 1e6, 1),
                          "fp6_same_bits": same})
    # the dual-uniform layer (input columns 0..9 of the weights on a scale of their own): the reference's epilogue
    # (one launch after the quantizer) and the row-sum mode that splits the accumulator at column 10 (quantizer,
    # GEMM into int32, epilogue)
    dual_rowsum = LinearQuant4bitDUASQRowSum.from_linear(lin)
    dual_ref = LinearQuant4bitDUASQ.from_linear(lin.cpu()).to(dev)
    for name, mod in (("dual_reference_mode", dual_ref), ("dual_rowsum_mode", dual_rowsum)):
        us = graph_time_us([lambda: mod(x)] * 20)
        y = mod(x).float()
        out[name] = {"step_us": round(us, 2), "TOPS": round(2.0 * M * N * K / us / 1e6, 1),
                     "rel_error_vs_fp32_matmul": round(float((y.detach() - true).norm() / true.norm()), 4)}
    return out


def other_shapes_section(dev):
    """The other prefill shapes of the Llama-2-7B configuration and the Llama-2-70B MLP shapes at M = 4096 (a full
    layer on one GPU): one module step (quantize + GEMM + dequant) on either matrix path, HIP-graph timed."""
    import torch

    from duqlinear4bitcuda_amd.nn import Linear4bitSQ, SymQuantizer

    out = []
    for (M, K, N) in [(2048, 4096, 11008), (2048, 11008, 4096), (4096, 8192, 28672), (4096, 28672, 8192)]:
        x = heavy_tail_acts(M, K, seed=5).to(dev)
        w, sw = random_weights(N, K, seed=55, dev=dev)
        lin = Linear4bitSQ(K, N, bias=False).to(dev)
        lin.weight.copy_(w)
        lin.weight_scales = sw
        q_i8 = SymQuantizer(1.0)
        q_f6 = SymQuantizer(1.0, shadow="only", shadow_min_rows=1)
        reps = 6 if M * N * K < 2e11 else 3
        us_i8 = graph_time_us([lambda: lin(q_i8(x))] * reps)
        y_i8 = lin(q_i8(x))
        lin.enable_fp6()
        same = bool(torch.equal(lin(q_f6(x)).view(torch.int16), y_i8.view(torch.int16)))
        us_f6 = graph_time_us([lambda: lin(q_f6(x))] * reps)
        ops = 2.0 * M * N * K
        out.append({"M": M, "K": K, "N": N, "integer_step_us": round(us_i8, 1), "integer_TOPS": round(ops / us_i8 / 1e6, 1),
                    "fp6_step_us": round(us_f6, 1), "fp6_TOPS": round(ops / us_f6 / 1e6, 1), "same_bits": same})
        del lin, w, x
    return out


def batched_section(dev, quick=False):
    """Quantized activation x activation products at attention-like shapes (AsymQuantMatMul, n = 32 heads): scores
    Q K^T (HA = HB = 2048 tokens, W = 128) and P V (HA = 2048, HB = 128, W = 2048).  HIP-graph timed: the fused
    batched launch, the reference's two steps as two batched launches (GEMM into int32, batched dequant), one fused
    launch per batch entry (what a loop over the single-problem entry point costs on the GPU alone, without the
    host time of n launches), and the whole module (two quantizers + the fused launch)."""
    import torch

    from duqlinear4bitcuda_amd import _HIP as hip
    from duqlinear4bitcuda_amd.nn import AsymQuantMatMul

    out = []
    for (n, HA, HB, W) in [(32, 2048, 2048, 128)] if quick else [(32, 2048, 2048, 128), (32, 2048, 128, 2048),
                                                                  (32, 1, 2048, 128)]:
        a = torch.randn(n, HA, W, device=dev).half()
        b = torch.randn(n, HB, W, device=dev).half()
        mod = AsymQuantMatMul()
        qa, qb = mod.quantizer_A(a), mod.quantizer_B(b)
        args = (hip.EPI_ASYM, qa.quantized_x, qa.scales_x, qa.zeros_x, qb.quantized_x, qb.scales_x, qb.zeros_x)
        us_fused = graph_time_us([lambda: hip.batch_linear4bit_forward(*args)] * 6)
        acc = hip.batched_matmul(qa.quantized_x, qb.quantized_x)
        us_mm = graph_time_us([lambda: hip.batched_matmul(qa.quantized_x, qb.quantized_x)] * 6)
        us_dq = graph_time_us([lambda: hip.asym_batch_dequant(acc, qa.scales_x, qa.zeros_x, qb.scales_x, qb.zeros_x)] * 6)

        def loop():
            for i in range(n):
                hip.linear4bit_forward(hip.EPI_ASYM, qa.quantized_x[i], qa.scales_x[i], qa.zeros_x[i], qb.quantized_x[i],
                                       qb.scales_x[i], qb.zeros_x[i])

        us_loop = graph_time_us([loop] * 3)
        us_mod = graph_time_us([lambda: mod(a, b)] * 6)
        ops = 2.0 * n * HA * HB * W
        byts = n * (HA * W // 2 + HB * W // 2 + 4 * (HA + HB) + 2 * HA * HB)
        out.append({"n": n, "HA": HA, "HB": HB, "W": W, "fused_us": round(us_fused, 2),
                    "fused_TOPS": round(ops / us_fused / 1e6, 1), "fused_GBps": round(byts / us_fused / 1e3, 1),
                    "fused_frac_hbm": round(byts / us_fused / 1e3 / PEAK_HBM_GBS, 4),
                    "batched_matmul_int32_us": round(us_mm, 2), "asym_batch_dequant_us": round(us_dq, 2),
                    "per_entry_launches_us": round(us_loop, 2), "module_us": round(us_mod, 2)})
        del a, b, acc
    return out


def stack_section(dev):
    """A stack of eight Sequential(SymQuantizer, Linear4bitSQ) layers of 4096 x 4096 (a decode step through eight
    projections): wall time per step called eagerly and replayed as one HIP graph (tools.graphs.GraphedForward;
    the graphed figure includes the copy of the input into the recording and the replay's launch)."""
    import torch

    from duqlinear4bitcuda_amd.nn import Linear4bitSQ, SymQuantizer
    from duqlinear4bitcuda_amd.tools.graphs import GraphedForward

    K = N = 4096
    g = torch.Generator().manual_seed(9)
    layers = []
    for _ in range(8):
        layer = Linear4bitSQ(K, N, bias=False).to(dev)
        layer.weight = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=g).to(dev)
        layer.weight_scales = (torch.rand(N, 1, generator=g) * 0.002 + 0.0005).half().to(dev)
        layers += [SymQuantizer(1.0), layer]
    model = torch.nn.Sequential(*layers)
    out = []
    for M in (1, 4, 16):
        x = torch.randn(1, M, K, generator=g).half().to(dev)
        graphed = GraphedForward(model, x)
        same = bool(torch.equal(graphed(x).view(torch.int16), model(x).view(torch.int16)))
        out.append({"layers": 8, "M": M, "K": K, "N": N, "eager_us_per_step": round(eager_wall_us([model], x, steps=300, warm=50), 2),
                    "graphed_us_per_step": round(eager_wall_us([graphed], x, steps=300, warm=50), 2), "same_bits": same})
    return out


def int8_layer_section(dev, quick=False):
    """The 8-bit asymmetric layer (LinearQuant8bitASQ) at the headline shape: float32 activations, quantizer
    launch + fused GEMM launch, float32 result; the GEMM alone against the dense int8 MFMA peak."""
    import torch

    from duqlinear4bitcuda_amd import _HIP
    from duqlinear4bitcuda_amd.nn import LinearQuant8bitASQ

    out = []
    for (M, K, N) in [(2048, 4096, 4096)] if quick else [(2048, 4096, 4096), (2048, 4096, 11008), (16, 4096, 4096)]:
        g = torch.Generator().manual_seed(6)
        x = torch.randn(M, K, generator=g).to(dev)
        layer = LinearQuant8bitASQ(K, N, bias=False).to(dev)
        layer.weight.copy_(torch.randint(0, 128, (N, K), dtype=torch.int8, generator=g))
        layer.weight_scales.copy_(torch.rand(N, 1, generator=g) * 0.009 + 0.001)
        layer.weight_zeros.copy_(-torch.randint(0, 20, (N, 1), generator=g).float())
        p = layer.quantizer(x)
        y = layer(x)
        layer.fused = False
        same = bool(torch.equal(layer(x), y))     # the reference's three steps give the same bits
        us3 = graph_time_us([lambda: layer(x)] * 10)
        layer.fused = True
        ops = 2.0 * M * N * K
        us_step = graph_time_us([lambda: layer(x)] * 10)
        wt = layer._tiled_weight()
        us_gemm = graph_time_us([lambda: _HIP.linear8bit_forward(p.quantized_x, p.scales_x, p.zeros_x, wt,
                                                                 layer.weight_scales, layer.weight_zeros,
                                                                 tiled_rows=N)] * 10)
        us_rowmajor = graph_time_us([lambda: _HIP.linear8bit_forward(p.quantized_x, p.scales_x, p.zeros_x, layer.weight,
                                                                     layer.weight_scales, layer.weight_zeros)] * 10)
        us_quant = graph_time_us([lambda: layer.quantizer(x)] * 10)
        eager = {}
        if M <= 256:  # a step of a few rows is bound by the host: one library call (the default) against two
            eager["module_eager_us"] = round(eager_wall_us([layer], x), 2)
            layer.one_call_rows = 0
            eager["module_eager_two_calls_us"] = round(eager_wall_us([layer], x), 2)
            layer.one_call_rows = 1024
        out.append({"M": M, "K": K, "N": N, "step_us": round(us_step, 2), "step_TOPS": round(ops / us_step / 1e6, 1), **eager,
                    "three_step_us": round(us3, 2), "fused_equals_three_steps": same,
                    "quantize_us": round(us_quant, 2),
                    "quantize_GBps": round((M * K * 5 + M * 8) / us_quant / 1e3, 1),
                    "gemm_rowmajor_weight_us": round(us_rowmajor, 2),
                    "gemm_fused_us": round(us_gemm, 2), "gemm_TOPS": round(ops / us_gemm / 1e6, 1),
                    "gemm_frac_of_int8_peak": round(ops / us_gemm / 1e6 / PEAK_INT8_TOPS, 4),
                    "gemm_algorithmic_GBps": round((M * K + N * K + M * N * 4) / us_gemm / 1e3, 1)})
        del layer, x
    if quick:
        return out
    # decode: weights rotated over more than 512 MB of distinct buffers, as in decode_section
    decode = []
    for (M, K, N) in [(1, 4096, 4096), (4, 4096, 4096), (1, 4096, 11008), (16, 4096, 4096), (16, 4096, 11008),
                      (32, 4096, 11008)]:
        g = torch.Generator().manual_seed(7)
        nbuf = int(600e6 // (N * K)) + 1
        w0 = torch.randint(0, 128, (N, K), dtype=torch.int8, generator=g).to(dev)
        # like the layer: up to four rows read `weight` itself (rows kernel), more read its tiled copy
        few = M <= 4
        ws = [torch.roll(w0, i, 0).contiguous() if few else _HIP.weight_tile_8bit(torch.roll(w0, i, 0)) for i in range(nbuf)]
        q = torch.randint(0, 127, (M, K), dtype=torch.int8, generator=g).to(dev)
        sx, zx = torch.rand(M, 1, device=dev) + 0.1, torch.zeros(M, 1, device=dev)
        sw, zw = torch.rand(N, 1, device=dev) * 0.01, torch.zeros(N, 1, device=dev)
        us = graph_time_us([(lambda w=w: _HIP.linear8bit_forward(q, sx, zx, w, sw, zw, tiled_rows=None if few else N))
                            for w in ws] * 2)
        us_read = graph_time_us([(lambda w=w: _HIP.probe_read(w)) for w in ws] * 2)
        byts = M * K + N * K + 8 * N + 8 * M + 4 * M * N
        decode.append({"M": M, "K": K, "N": N, "gemm_fused_us": round(us, 3), "GBps": round(byts / us / 1e3, 1),
                       "frac_hbm": round(byts / us / 1e3 / PEAK_HBM_GBS, 4), "read_floor_us": round(us_read, 3),
                       "frac_of_read_floor": round(us_read / us, 4), "weight": "row-major" if few else "tiled copy",
                       "weight_buffers": nbuf})
        del ws, w0
    out.append({"decode_rotated_weights": decode})
    return out


def cpu_baseline(x_cpu, wq_cpu, sw_cpu, ops, budget_s=15.0):
    """The reference's CPU fake-quant path (torch-CPU) on the same workload, host cores: whole forwards repeated for
    about budget_s seconds."""
    import torch

    from oracle import fakequant_torch as fq

    fq.linear4bit_forward(x_cpu[:64], wq_cpu, sw_cpu)  # warm
    t0 = time.perf_counter()
    reps = 0
    while True:
        fq.linear4bit_forward(x_cpu, wq_cpu, sw_cpu)
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= 400:
            break
    per = el / reps
    return {"value": round(ops / per / 1e12, 4), "unit": "TOPS", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"full workload, {reps} reps of torch-CPU fake-quant forward (fp32 matmul of integer codes), "
                      f"{per * 1e3:.1f} ms each, os.cpu_count()={os.cpu_count()}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=300)
    ap.add_argument("--quick", action="store_true", help="skip the larger decode shapes and shorten the CPU baseline")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-harness", action="store_true",
                    help="skip the eager wall-clock sections (the reference's harness table, the modules' eager decode "
                         "figures): for runs under a profiler, where every launch is slow")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists or is measured)",
              file=sys.stderr)
        sys.exit(2)

    import torch

    from duqlinear4bitcuda_amd import _HIP as hip
    from duqlinear4bitcuda_amd import _lib
    from duqlinear4bitcuda_amd.nn import Linear4bitSQ, SymQuantizer
    from duqlinear4bitcuda_amd.tools import unpack_i4

    _lib.load()
    dev = torch.device("cuda:0")
    M, N, K = 2048, 4096, 4096
    ops = 2.0 * M * N * K

    x_cpu = heavy_tail_acts(M, K, seed=3)
    x = x_cpu.to(dev)
    w, sw = random_weights(N, K, seed=33, dev=dev)
    lin = Linear4bitSQ(K, N, bias=False).to(dev)
    lin.weight.copy_(w)
    lin.weight_scales = sw
    lin.enable_fp6()
    quant = SymQuantizer(1.0, shadow="only", shadow_min_rows=1)
    lin_i8 = Linear4bitSQ(K, N, bias=False).to(dev)   # the same layer on the i8 MFMA kernels
    lin_i8.weight.copy_(w)
    lin_i8.weight_scales = sw
    quant_i8 = SymQuantizer(1.0)

    def step():
        return lin(quant(x))

    def step_i8():
        return lin_i8(quant_i8(x))

    if not torch.equal(step().view(torch.int16), step_i8().view(torch.int16)):
        raise SystemExit("bench.py: the 6-bit float path and the integer path disagree")

    # ---- whole-step throughput: W warm-up steps, then exactly K timed steps ----
    # (before them, untimed, enough steps to bring the part to the clock it holds under this load: after an idle
    # period that takes about a millisecond, and a short run would otherwise measure the ramp)
    for _ in range(PREWARM_STEPS + args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    tops = ops / (ms_per_step * 1e-3) / 1e12

    # the same K steps recorded once into a HIP graph: untimed replays for about 10 ms (the W warm-up steps and the
    # clock ramp), then ONE timed replay = exactly K steps, bracketed by synchronize() like the eager loop
    graph_ms_per_step = None
    try:
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            step()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(args.steps):
                step()
        for _ in range(max(2, int(10.0 / max(ms_per_step * args.steps, 1e-3)))):
            g.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        g.replay()
        torch.cuda.synchronize()
        graph_ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
        del g
    except RuntimeError as exc:  # capture unsupported: keep the eager figure only
        print(f"graph capture skipped: {exc}", file=sys.stderr)
    # `value` is the eager module path, which is how the reference's own harness times a layer
    # (test/benchmark.py:24-39); the graph replay of the same K steps is reported beside it
    eager_ms_per_step = ms_per_step
    timed_path = "eager module calls"

    # ---- the same steps on the integer kernels ----
    for _ in range(PREWARM_STEPS + args.warmup):
        step_i8()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_i8()
    torch.cuda.synchronize()
    i8_ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- dominant kernel (fused GEMM + dequant) alone, HIP events on the launch stream ----
    pq = quant(x)
    xs, sx = pq.shadow_x, pq.scales_x
    n_timed = max(args.steps, EVENT_TIMED_LAUNCHES)
    with ClockSampler() as clk_f6:
        gemm_us = event_time_us(lambda: hip.linear4bit_forward_bf6(hip.EPI_SYM, xs, sx, None, lin.weight_shadow, sw),
                                n_timed, PREWARM_STEPS + args.warmup)
    # the quantizer takes less time than a launch from Python: replayed from a HIP graph instead
    quant_us = graph_time_us([lambda: hip.quantize_rows_sym_bf6(x, with_q=False)] * 40)
    achieved = ops / gemm_us / 1e6
    roofline = {"bound": "mfma", "kernel": "gemm_bf6_kernel<8,4,0,false> (fused GEMM + dequant on v_mfma_f32_16x16x128_f8f6f4, 128 x 256 tiles)",
                "achieved": round(achieved, 1), "peak": PEAK_FP6_TOPS, "unit": "TOP/s",
                "frac": round(achieved / PEAK_FP6_TOPS, 4), "frac_of_int8_peak": round(achieved / PEAK_INT8_TOPS, 4),
                "avg_kernel_us": round(gemm_us, 2), "launches_timed": n_timed,
                # what the driver reported as the shader clock while those launches ran (pp_dpm_sclk): boxes of the
                # pool differ by a few per cent in the clock they hold, and avg_kernel_us with them
                "shader_clock_during_timing": clk_f6.summary(),
                "peak_note": "published dense fp6 peak; the same achieved rate is %.3f of the int8 peak (5.0 POP/s) the "
                             "integer kernel is priced against" % (achieved / PEAK_INT8_TOPS),
                # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this workload, each
                # scaled by what the counter reads for the 256 MiB copy at the end of this script
                "traffic": profile_traffic_bytes("gemm_bf6_kernel__prefill_M2048_K4096_N4096.txt", "gemm_bf6_kernel"),
                "traffic_source": "profiles/gemm_bf6_kernel__prefill_M2048_K4096_N4096.txt"}
    xq = quant_i8(x).quantized_x
    with ClockSampler() as clk_i8:
        i8_gemm_us = event_time_us(lambda: hip.linear4bit_forward(hip.EPI_SYM, xq, sx, None, lin_i8.weight, sw), n_timed,
                                   PREWARM_STEPS + args.warmup)
    i8_quant_us = graph_time_us([lambda: hip.quantize_rows_sym(x)] * 40)
    integer_path = {"ms_per_step": round(i8_ms_per_step, 5), "TOPS": round(ops / (i8_ms_per_step * 1e-3) / 1e12, 2),
                    "kernel": "gemm_s4_stream_kernel<4,0,false,2> (v_mfma_i32_32x32x32_i8, 128 x 256 tiles)", "gemm_fused_us": round(i8_gemm_us, 2),
                    "quantize_rows_sym_us": round(i8_quant_us, 2),
                    "roofline": {"bound": "mfma", "kernel": "gemm_s4_stream_kernel (fused GEMM + dequant on v_mfma_i32_32x32x32_i8)",
                                 "achieved": round(ops / i8_gemm_us / 1e6, 1), "peak": PEAK_INT8_TOPS,
                                 "unit": "TOP/s", "frac": round(ops / i8_gemm_us / 1e6 / PEAK_INT8_TOPS, 4),
                                 "avg_kernel_us": round(i8_gemm_us, 2), "launches_timed": n_timed,
                                 "shader_clock_during_timing": clk_i8.summary(),
                                 "traffic": profile_traffic_bytes("gemm_s4_stream_kernel__prefill_M2048_K4096_N4096.txt",
                                                                  "gemm_s4_stream_kernel"),
                                 "traffic_source": "profiles/gemm_s4_stream_kernel__prefill_M2048_K4096_N4096.txt"}}
    # the driver record keeps `roofline`: the integer path's figures ride inside it as a second entry
    roofline["integer_path"] = integer_path["roofline"]

    decode = decode_section(dev, args.quick, eager=not args.no_harness)
    quantizer = quantizer_section(dev)
    asym = None if args.quick else asym_section(dev)
    other = None if args.quick else other_shapes_section(dev)
    int8_layer = int8_layer_section(dev, args.quick)
    batched = batched_section(dev, args.quick)
    harness = None if args.no_harness else harness_section(dev, args.quick)
    fanout = None if args.quick else fanout_section(dev)
    stack = None if args.quick or args.no_harness else stack_section(dev)
    rows_7b = [d for d in decode if (d["M"], d["N"], d["K"]) in LLAMA7B_DECODE]
    worst = min(rows_7b, key=lambda d: d["frac_hbm"])
    roofline_decode = {"bound": "hbm", "kernel": "gemv_s4_rows_kernel (M <= 8, quantizer inside) / quantize_rows_kernel + "
                                                 "gemm_s4_decode_kernel (M <= 64)",
                       "what": "worst of the Llama-2-7B decode rows (M in {1,4,16}, K=4096, N in {4096,11008}), binary16 "
                               "activations in, quantize + GEMM + dequant, weights never in a cache",
                       "achieved": worst["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": worst["frac_hbm"],
                       "shape": {k: worst[k] for k in ("M", "N", "K")},
                       "best_7b_frac": max(d["frac_hbm"] for d in rows_7b),
                       "read_floor_frac": round(worst["read_floor_GBps"] / PEAK_HBM_GBS, 4),
                       # the GEMM launch of that row (the quantizer launch of 16 rows before it moves 0.2 MB)
                       "traffic": profile_shape_traffic_bytes("decode_kernels__bench_shapes.txt", "gemm_s4_decode_kernel<8, 4, 0, 1,", 256)
                       if (worst["M"], worst["N"]) == (16, 4096) else None,
                       "traffic_source": "profiles/decode_kernels__bench_shapes.txt"}

    cpu = None
    if not args.no_cpu:
        wq_cpu = unpack_i4(w.cpu()).float()
        cpu = cpu_baseline(x_cpu, wq_cpu, sw.cpu(), ops, budget_s=5.0 if args.quick else 15.0)

    # a device copy of known size: the reference point for scaling hardware byte counters
    # (FETCH_SIZE / WRITE_SIZE) when this script runs under rocprofv3 --pmc
    ref_src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
    ref_dst = torch.empty_like(ref_src)
    ref_dst.copy_(ref_src)
    torch.cuda.synchronize()

    props = torch.cuda.get_device_properties(0)
    line = {
        "metric": "int4 Linear TOPS (prefill) & HBM GB/s (decode) at Llama-7B shapes, 1 MI355X",
        "value": round(tops, 2), "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "prewarm_steps": PREWARM_STEPS,
        "ms_per_step": round(ms_per_step, 5),
        "graph_ms_per_step": None if graph_ms_per_step is None else round(graph_ms_per_step, 5),
        "eager_ms_per_step": round(eager_ms_per_step, 5), "timed_path": timed_path,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp6", "dtype_detail": "int4 x int4 codes held as E3M2 6-bit floats for v_mfma_f32_16x16x128_f8f6f4, float32 "
                                        "accumulate (exact: integers below 2^24), fp16 epilogue; bit-identical to the int8 path",
        "data": "synthetic",
        "config": {"workload": "prefill Linear4bit forward (quantize + GEMM + dequant), M=2048 K=4096 N=4096, "
                               "symmetric int4 both operands, activations ~N(0,1) with 1% Student-t(3) channels",
                   "M": M, "N": N, "K": K, "step_kernels": {"quantize_rows_sym_bf6_us": round(quant_us, 2),
                                                             "gemm_fused_us": round(gemm_us, 2)}},
        "roofline": roofline,
        "integer_path": integer_path,
        "roofline_decode": roofline_decode,
        "decode": decode,
        "quantizer": quantizer,
        "asym": asym,
        "other_shapes": other,
        "int8_layer": int8_layer,
        "batched": batched,
        "harness": harness,
        "fanout": fanout,
        "stack": stack,
        "cpu_baseline": cpu,
        "device": {"name": props.name, "arch": props.gcnArchName, "cus": props.multi_processor_count},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
