#!/usr/bin/env python3
"""Benchmark of the mixed INT4/FP6 weight-only GEMM on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]          one JSON line (the driver's contract)
    python bench.py --sweep sweep.json                           per-shape table for all benchmark configurations
    python bench.py --shape 128,8192,8192                        one shape (m,k,n[,quant_cols,group_size])
    python bench.py --models                                     the reference's own benchmark (bench.py:57-119): five models' layers at batch 16

Workload of the JSON line: decode (M=1) through Llama-2-7B layer shapes (K x N) 4096x12288, 4096x4096,
4096x22016, 11008x4096; INT4 with group-128 scales plus 256 FP6 columns.  A *step* is one layer: those four
GEMMs.  Eight distinct layers (8 x 105.7 MB of packed weights) are cycled so that neither the L2 nor the
256 MB Infinity Cache can serve the weight stream.  Packed words are random bits, scales random positive
fp16, activations N(0,1) fp16 (the reference's own bench does the same, bench.py:26-34).

value        packed-weight GB/s over the timed steps: algorithmic weight bytes / wall time, where
             weight bytes = K(N-qc)/2 + K*qc*3/4 + scale bytes.
roofline     the GEMM kernel against the 8 TB/s HBM peak: algorithmic bytes per launch / mean time per
             launch, measured with HIP events on the launch stream over the same timed region.
cpu_baseline the oracle's CPU path (quantise + prepack + dequantise-then-matmul) on config 0 (16 x 4096 x 4096), stage
             by stage, single-threaded like the reference (`value`) and on all cores, on this box's host cores.
Also reported: a fp16 torch.matmul (hipBLASLt/rocBLAS) over the same shapes and rotation, and the speed-up.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "fp6-marlin_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the headline workload (mean of its four GEMMs): FETCH_SIZE + WRITE_SIZE from two
# `rocprofv3 --pmc` runs of `bench.py --traffic-probe`, each scaled by what the same counter reads for a
# 256 MiB device copy (x2.000 and x1.000); figures in profiles/gemm_sk_kernel_decode7b_hbm_traffic.txt.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = 28742537
TRAFFIC_PROFILE = "profiles/gemm_sk_kernel_decode7b_hbm_traffic.txt"
MFMA_F16_PEAK_TFLOPS = 2500.0
LLAMA7B = [(4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096)]
LLAMA70B = [(8192, 10240), (8192, 8192), (8192, 57344), (28672, 8192)]


def weight_bytes(k, n, qc, gs):
    n4 = n - qc
    scale = 2 * n if gs == -1 else 2 * (k // gs) * n4 + 2 * qc
    return k * n4 // 2 + k * qc * 3 // 4 + scale


class Problem:
    """Device operands of one (m, k, n) GEMM with random packed words.  All problems share one workspace: the
    benchmark's calls run back to back on one stream (the library keeps a partial-sum region per workspace)."""
    shared_ws = None

    def __init__(self, torch, m, k, n, qc, gs, gen, fp16_ref=False, on_device=False):
        dev = torch.device("cuda:0")
        n4 = n - qc
        words = k * n4 // 8 + k * qc * 3 // 16
        self.m, self.k, self.n, self.qc, self.gs = m, k, n, qc, gs
        if on_device:                                                    # (layers of hundreds of MB: the host generator takes seconds)
            self.B = torch.randint(-2 ** 31, 2 ** 31 - 1, (words,), dtype=torch.int32, device=dev)
        else:
            self.B = torch.randint(-2 ** 31, 2 ** 31 - 1, (words,), generator=gen, dtype=torch.int64).to(torch.int32).to(dev)
        ns = (n4 if gs == -1 else (k // gs) * n4) + qc
        self.s = (torch.rand(ns, generator=gen) * 0.01 + 0.001).half().to(dev)
        self.A = torch.randn((m, k), generator=gen).half().to(dev)
        self.C = torch.zeros((m, n), dtype=torch.half, device=dev)
        if Problem.shared_ws is None:
            import fp6_marlin
            Problem.shared_ws = fp6_marlin.init_workspace(torch.zeros(65536, dtype=torch.int32, device=dev))
        assert n // 128 * 16 <= Problem.shared_ws.numel()
        self.ws = Problem.shared_ws
        self.W16 = (torch.randn((k, n), generator=gen) * 0.02).half().to(dev) if fp16_ref else None
        self.bytes = weight_bytes(k, n, qc, gs)
        self.flops = 2 * m * k * n

    def run(self, mul):
        mul(self.A, self.B, self.C, self.s, self.ws, self.qc if self.qc else -1, -1, -1, -1, 16, self.gs)

    def run_gfx950(self, mul_fused):
        """The same words read in the gfx950 order (random bits either way: the timing is what matters here)."""
        mul_fused(self.A, self.B, self.C, self.s, self.ws, self.qc if self.qc else -1, self.gs, layout="gfx950")

    def run_fp16(self, torch):
        torch.matmul(self.A, self.W16, out=self.C)


SETTLE_MS = 50.0


def settle(torch, fn, calls, ms=SETTLE_MS):
    """Replay the workload about to be timed for at least `ms` milliseconds (untimed) and return the number of calls.
    An MI355X that has been idle (tensor set-up on the host, graph capture) needs tens of milliseconds of the same kind
    of load to reach the clocks it sustains under it: measured on 8192 x 57344 at M=1, 50-58 us per launch right after
    an idle period against 43-45 us after 20 ms of the same launches (an unrelated fp16 matmul loop does not do it,
    and leaves the memory-bound launches slower).  Every timed region here -- the quantised GEMM and the fp16
    baseline alike -- starts from the steady state a serving loop is in."""
    n = 0
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for i in range(calls):
            fn(i)
        torch.cuda.synchronize()
        n += calls
    return n


def time_region(torch, fn, iters):
    """Wall clock (synchronised on both sides) and HIP-event time of `iters` calls of fn(i)."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for i in range(iters):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return t1 - t0, start.elapsed_time(stop) * 1e-3


def _median(fn, reps):
    ts = []
    out = None
    for _ in range(reps):
        t0 = time.perf_counter()
        out = fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2], out


def cpu_config0(torch, threaded):
    """The reference's CPU path on config 0 (M=16, K=4096, N=4096, 256 FP6 columns, INT4 g128), its five stages
    timed separately (median of five): (1) FP6 scale + clamp + cast (test.py:19-32, weight_quant.cpp:27-124),
    (2) FP6 2+4 prepack (weight_prepacking.cpp:123-177), (3) INT4 quantise + Marlin pack (test.py:85-121),
    (4) dequantise to the fp16 check weight (weight_prepacking.cpp:180-217, test.py:98), (5) the matmul on the CPU
    (fp32, the fp16 inputs are exact in it).  threaded=False: the oracle's restatement on one thread, as the reference
    runs (weight_quant.cpp:114 has its OpenMP pragma commented out); threaded=True: this package's own host
    routines and torch on all cores."""
    import numpy as np
    m, k, n, qc, gs = 16, 4096, 4096, 256, 128
    g = torch.Generator().manual_seed(0)
    a = torch.randn((m, k), generator=g).half()
    w = (torch.randn((k, n), generator=g) * 0.02).half()
    w4, w6 = w[:, : n - qc].contiguous(), w[:, n - qc:].contiguous()
    if threaded:
        from fp6_marlin import cabi as api
        asnp = lambda t: t                                               # (the package's routines take tensors)
    else:
        from oracle import fp6m_oracle as api
        asnp = lambda t: t.numpy()

    def fp6_cast():
        s = torch.max(torch.abs(w6), 0, keepdim=True)[0]
        s *= 1.0 / 28.0
        s = s.reshape(-1)
        x = w6 / s
        x = torch.where(torch.abs(x) < 0.0625, torch.zeros_like(x), x)
        x = torch.clamp(x, -28.0, 28.0)
        return api.fp6_quantize(asnp(x)), s

    t1, (q6, s6) = _median(fp6_cast, 5)
    t2, _ = _median(lambda: api.fp6_prepack(q6), 5)

    def int4():
        codes, s, ref = api.int4_quantize(asnp(w4), gs)
        return api.int4_pack(codes), codes, s

    t3, (_, codes, s4) = _median(int4, 5)

    def dequant():
        r6 = api.fp6_dequant(q6, asnp(s6))
        r6 = torch.as_tensor(r6).t()
        c = torch.as_tensor(codes).float() - 8.0
        r4 = (c.reshape(k // gs, gs, n - qc) * torch.as_tensor(s4).float().reshape(k // gs, 1, n - qc)).reshape(k, n - qc).half()
        return torch.cat([r4, r6], dim=1).contiguous()

    t4, w_ref = _median(dequant, 5)
    t5, _ = _median(lambda: torch.matmul(a.float(), w_ref.float()), 5)
    total = t1 + t2 + t3 + t4 + t5
    nbytes = weight_bytes(k, n, qc, gs)
    return {"seconds": round(total, 4), "GBs": round(nbytes / total / 1e9, 4),
            "stages_s": {"fp6_scale_clamp_cast": round(t1, 4), "fp6_prepack": round(t2, 4), "int4_quantise_pack": round(t3, 4),
                         "dequantise": round(t4, 4), "matmul_fp32": round(t5, 5)},
            "torch_threads": torch.get_num_threads()}


def cpu_baseline(torch):
    """The reference's CPU path restated (oracle/), timed on this box's host cores: config 0 stage by stage, on one
    thread (`value`; the reference is single-threaded) and on all cores (this package's threaded host routines),
    and one layer of the headline workload (decode M=1, the four Llama-2-7B shapes) on one thread."""
    import numpy as np
    from oracle import fp6m_oracle as oracle
    threads = torch.get_num_threads()
    torch.set_num_threads(1)
    try:
        one = cpu_config0(torch, threaded=False)
    finally:
        torch.set_num_threads(threads)
    many = cpu_config0(torch, threaded=True)
    m, qc, gs = 1, 256, 128
    torch.set_num_threads(1)
    t_prep = t_mm = 0.0
    nbytes = 0
    try:
        rng = np.random.default_rng(0)
        for k, n in LLAMA7B:
            w = rng.normal(0, 0.02, (k, n)).astype(np.float16)
            a = rng.normal(0, 1, (m, k)).astype(np.float16)
            t0 = time.perf_counter()
            w_ref, b, s = oracle.gen_mixed_weight(w, qc, gs)    # quantise, dequantise (w_ref), pack, prepack
            t1 = time.perf_counter()
            c = torch.matmul(torch.from_numpy(a).float(), torch.from_numpy(w_ref).float())
            t2 = time.perf_counter()
            t_prep += t1 - t0
            t_mm += t2 - t1
            nbytes += weight_bytes(k, n, qc, gs)
            del c, b, s, w_ref
    finally:
        torch.set_num_threads(threads)
    return {"value": one["GBs"], "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "config 0 (M=16, K=4096, N=4096, 256 FP6 columns, INT4 g128; 8,897,024 packed weight bytes): quantise + "
                      "prepack + dequantise + fp32 matmul, medians of five per stage, the oracle's restatement on one thread",
            "one_thread": one, "all_cores": dict(many, cores=os.cpu_count(), kind="this package's threaded host routines + torch"),
            "os_cpu_count": os.cpu_count(), "torch_num_threads": threads,
            "headline_layer_one_thread": {
                "GBs": round(nbytes / (t_prep + t_mm) / 1e9, 4), "weight_bytes": nbytes,
                "quantise_prepack_dequantise_s": round(t_prep, 2), "matmul_fp32_s": round(t_mm, 3),
                "sample": "one layer of the headline workload (M=1, the four Llama-2-7B shapes, INT4 g128 + 256 FP6 columns)"}}


# Layer sets of the reference's own benchmark (bench.py:57-85: k x n per layer) and what its chart shows for them at
# batch 16 on an RTX 4090D (assets/models.png, read off the bars: all INT4 / INT4 + 256 FP6 columns).
REFERENCE_MODELS = {
    "Llama7B": [(4096, 3 * 4096), (4096, 4096), (4096, 2 * 10752), (10752, 4096)],
    "Llama13B": [(5120, 3 * 5120), (5120, 5120), (5120, 2 * 13568), (13568, 5120)],
    "Llama33B": [(6656, 3 * 6656), (6656, 6656), (6656, 2 * 17664), (17664, 6656)],
    "Llama65B": [(8192, 3 * 8192), (8192, 8192), (8192, 2 * 21760), (21760, 8192)],
    "Falcon180B": [(14848, 14848 * 5 + 1024), (14848 * 5, 14848)],
}
REFERENCE_CHART_4090D = {"Llama7B": (3.89, 3.73), "Llama13B": (4.10, 4.01), "Llama33B": (3.80, 3.77),
                         "Llama65B": (3.84, 3.78), "Falcon180B": (3.88, 3.84)}


def reference_models(torch, fp6_marlin, gen, calls_target=40):
    """The reference's published measurement (bench.py:57-85, 100-119): batch 16, per-channel scales, quant_cols -1 and
    256, over each model's layers; speed-up = total fp16 time / total time of the quantised GEMMs (its time-weighted
    mean of the per-layer speed-ups).  Timing protocol as everywhere here (HIP graphs over > 640 MB of rotated
    weights), not the reference's 100 calls on one weight."""
    rows = []
    for model, layers in REFERENCE_MODELS.items():
        for j, qc in enumerate((0, 256)):
            per = [measure_shape(torch, fp6_marlin, gen, model, 16, k, n, qc, -1, calls_target=calls_target, on_device=True)
                   for k, n in layers]
            t, t16 = sum(r["us"] for r in per), sum(r["fp16_us"] for r in per)
            nbytes = sum(weight_bytes(k, n, qc, -1) for k, n in layers)
            rows.append({"tag": f"reference bench {model} M=16 quant_cols={qc if qc else -1} group_size=-1", "m": 16,
                         "layers": [f"{k}x{n}" for k, n in layers], "us": round(t, 2), "fp16_us": round(t16, 2),
                         "speedup_vs_fp16": round(t16 / t, 2), "weight_GBs": round(nbytes / t / 1e3, 1),
                         "hbm_frac": round(nbytes / t / 1e3 / HBM_PEAK_GBS, 4),
                         "layer_us": [r["us"] for r in per], "layer_fp16_us": [r["fp16_us"] for r in per],
                         "reference_chart_speedup_rtx4090d": REFERENCE_CHART_4090D[model][j]})
    return rows


def graphed(torch, step, layers, steps):
    """fn(i) for time_region that replays HIP graphs of `layers` consecutive steps (launch-bound loops belong in
    graphs); steps that do not fill a whole graph are replayed from a second, shorter graph, so that every timed
    step runs the same way."""
    whole, rest = divmod(steps, layers)
    graph = None
    if whole:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(layers):
                step(i)
    tail = None
    if rest:
        tail = torch.cuda.CUDAGraph()
        with torch.cuda.graph(tail):
            for i in range(rest):
                step(i)

    def run(i):
        (graph if i < whole else tail).replay()
    return run, whole + (1 if rest else 0)


def headline(args):
    import torch
    import fp6_marlin
    gen = torch.Generator().manual_seed(0)
    qc, gs, m, layers = 256, 128, 1, 8
    fp6_marlin.init(0)
    model = [[Problem(torch, m, k, n, qc, gs, gen, fp16_ref=True) for (k, n) in LLAMA7B] for _ in range(layers)]
    step_bytes = sum(p.bytes for p in model[0])
    launches_per_step = len(LLAMA7B)

    def step(i):
        for p in model[i % layers]:
            p.run(fp6_marlin.mul)

    def step_fp16(i):
        for p in model[i % layers]:
            p.run_fp16(torch)

    # (graphs are captured before the warm-up steps: capturing leaves the GPU idle for milliseconds, and the first
    # launches after that run slower)
    if args.warmup:
        step(0)                                                          # (the first of the warm-up steps loads the kernels)
        torch.cuda.synchronize()
    fn, calls = (step, args.steps) if args.no_graph else graphed(torch, step, layers, args.steps)
    for i in range(1, args.warmup):
        step(i)
    settled = settle(torch, fn, calls)
    wall, ev = time_region(torch, fn, calls)
    step_fp16(0)
    torch.cuda.synchronize()
    fn16, calls16 = (step_fp16, args.steps) if args.no_graph else graphed(torch, step_fp16, layers, args.steps)
    for i in range(1, max(2, args.warmup // 4)):
        step_fp16(i)
    settle(torch, fn16, calls16)
    wall16, _ = time_region(torch, fn16, calls16)

    gbs = step_bytes * args.steps / wall / 1e9
    per_launch = ev / (args.steps * launches_per_step)
    achieved = step_bytes / launches_per_step / per_launch / 1e9
    out = {
        "metric": "weight-stream GB/s (M=1-16), TFLOP/s (M=128), speedup vs fp16 hipBLASLt",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "warmup_settle": f"after the {args.warmup} warm-up steps the same steps were replayed untimed for {SETTLE_MS:.0f} ms "
                         f"({settled} graph replays) so that the clocks are those of a running serving loop",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "decode M=1, Llama-2-7B layer shapes 4096x12288 4096x4096 4096x22016 11008x4096, "
                               "INT4 g128 + 256 FP6 columns, one step = one layer (4 GEMMs), 8 layers cycled",
                   "m": m, "quant_cols": qc, "group_size": gs, "weight_bytes_per_step": step_bytes},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs recorded in " + TRAFFIC_PROFILE +
                                       ", not measured in this run",
                     "kernel": "fp6m::gemm_sk_kernel<true, 0, false, false>", "us_per_launch": round(per_launch * 1e6, 3),
                     "bytes_per_launch": step_bytes // launches_per_step},
        "cpu_baseline": cpu_baseline(torch),
        "fp16_hipblaslt": {"ms_per_step": round(wall16 / args.steps * 1e3, 5),
                           "GBs": round(sum(2 * k * n for k, n in LLAMA7B) * args.steps / wall16 / 1e9, 1),
                           "speedup": round(wall16 / wall, 3)},
    }
    del model
    torch.cuda.empty_cache()
    # the other regimes the metric names (same protocol as --sweep): the 70B layer shapes at M = 1 and 16 and
    # the batch sweep on 8192 x 8192, each next to the fp16 GEMM of the same shape
    if not args.headline_only:
        regimes = [(f"70B M={mm}", mm, k, n) for mm in (1, 16) for (k, n) in LLAMA70B]
        regimes += [("7B M=16", 16, k, n) for (k, n) in LLAMA7B]
        regimes += [(f"batch sweep M={mm}", mm, 8192, 8192) for mm in (2, 4, 8, 32, 64, 128, 256, 512, 1024)]
        out["other_regimes"] = [measure_shape(torch, fp6_marlin, gen, tag, mm, k, n, qc, gs, calls_target=60)
                                for tag, mm, k, n in regimes]
        out["other_regimes"] += reference_models(torch, fp6_marlin, gen)
    print(json.dumps(out), flush=True)


def traffic_probe():
    """Work for a counter run: a plain copy of known size calibrates FETCH_SIZE / WRITE_SIZE (both must read
    256 MiB for it), then the four headline GEMMs run three times over distinct weights."""
    import torch
    import fp6_marlin
    gen = torch.Generator().manual_seed(0)
    fp6_marlin.init(0)
    src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    probs = [[Problem(torch, 1, k, n, 256, 128, gen) for (k, n) in LLAMA7B] for _ in range(3)]
    torch.cuda.synchronize()
    dst.copy_(src)
    for layer in probs:
        for p in layer:
            p.run(fp6_marlin.mul)
    torch.cuda.synchronize()
    print("traffic probe done: copy of", src.numel(), "bytes; GEMM weight bytes per launch",
          [p.bytes for p in probs[0]], flush=True)


def measure_shape(torch, fp6_marlin, gen, tag, m, k, n, qc, gs, calls_target=100, layout="reference", on_device=False):
    """One (m, k, n) GEMM against fp16 torch.matmul (hipBLASLt), both replayed from HIP graphs that walk
    over > 512 MB of distinct weights."""
    nbytes = weight_bytes(k, n, qc, gs)
    copies = max(2, min(24, int(640e6 // nbytes) + 1))
    probs = [Problem(torch, m, k, n, qc, gs, gen, on_device=on_device) for _ in range(copies)]
    n16 = max(2, min(copies, int(640e6 // (2 * k * n)) + 1))
    if on_device:
        w16 = [(torch.randn((k, n), device="cuda") * 0.02).half() for _ in range(n16)]
    else:
        w16 = [(torch.randn((k, n), generator=gen) * 0.02).half().cuda() for _ in range(n16)]

    def f(i):
        if layout == "gfx950":
            probs[i % copies].run_gfx950(fp6_marlin.mul_fused)
        else:
            probs[i % copies].run(fp6_marlin.mul)

    def f16(i):
        torch.matmul(probs[0].A, w16[i % len(w16)], out=probs[0].C)

    f(0)                                                                 # (first call: scratch region, lazy module load)
    f16(0)
    torch.cuda.synchronize()
    iters, iters16 = copies * max(1, calls_target // copies), len(w16) * max(1, calls_target // len(w16))
    fn, calls = graphed(torch, f, copies, iters)
    fn16, calls16 = graphed(torch, f16, len(w16), iters16)
    settle(torch, fn, calls)                                             # warm-up right before each timed region
    _, ev = time_region(torch, fn, calls)
    settle(torch, fn16, calls16)
    _, ev16 = time_region(torch, fn16, calls16)
    t, t16 = ev / iters, ev16 / iters16
    row = {"tag": tag, "m": m, "k": k, "n": n, "quant_cols": qc, "group_size": gs, "layout": layout, "us": round(t * 1e6, 2),
           "weight_GBs": round(nbytes / t / 1e9, 1), "hbm_frac": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4),
           "TFLOPs": round(2 * m * k * n / t / 1e12, 2), "mfma_frac": round(2 * m * k * n / t / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
           "fp16_us": round(t16 * 1e6, 2), "fp16_GBs": round(2 * k * n / t16 / 1e9, 1), "speedup_vs_fp16": round(t16 / t, 2)}
    del probs, w16
    torch.cuda.empty_cache()
    return row


def one_shape(args):
    """`--shape m,k,n[,quant_cols,group_size]`: one JSON row for one shape (used for profiles of the m > 16 kernel)."""
    import torch
    import fp6_marlin
    v = [int(x) for x in args.shape.split(",")]
    m, k, n = v[:3]
    qc, gs = (v[3] if len(v) > 3 else 256), (v[4] if len(v) > 4 else 128)
    fp6_marlin.init(0)
    row = measure_shape(torch, fp6_marlin, torch.Generator().manual_seed(0), "shape", m, k, n, qc, gs, layout=args.layout)
    bound = "mfma" if m >= 128 else "hbm"
    row["roofline"] = ({"bound": "mfma", "achieved": row["TFLOPs"], "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                        "frac": row["mfma_frac"]} if bound == "mfma" else
                       {"bound": "hbm", "achieved": row["weight_GBs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": row["hbm_frac"]})
    print(json.dumps(row), flush=True)


def fused_bench(args):
    """`--fused m,k,n[,quant_cols,group_size]`: `mul_fused` (activation gather, output scatter, bias, residual in
    the call) against the same work done around `mul` with torch kernels; every variant replayed from a HIP
    graph over rotated weights."""
    import torch
    import fp6_marlin
    v = [int(x) for x in args.fused.split(",")]
    m, k, n = v[:3]
    qc, gs = (v[3] if len(v) > 3 else 256), (v[4] if len(v) > 4 else 128)
    gen = torch.Generator().manual_seed(0)
    fp6_marlin.init(0)
    copies = max(2, min(24, int(640e6 // weight_bytes(k, n, qc, gs)) + 1))
    probs = [Problem(torch, m, k, n, qc, gs, gen) for _ in range(copies)]
    a_cols = torch.randperm(k, generator=gen).to(torch.int32).cuda()
    c_cols = torch.randperm(n, generator=gen).to(torch.int32).cuda()
    # the map a Layer with chosen FP6 output features uses: the other features in order, then the chosen ones
    picked = torch.randperm(n, generator=gen)[:qc if qc else 256].sort().values
    keep = torch.ones(n, dtype=torch.bool)
    keep[picked] = False
    c_layer = torch.cat([torch.nonzero(keep).reshape(-1), picked]).to(torch.int32).cuda()
    inv = torch.argsort(c_cols.long())
    bias = torch.randn(n, generator=gen).half().cuda()
    res = torch.randn((m, n), generator=gen).half().cuda()
    out = torch.empty((m, n), dtype=torch.half, device="cuda")
    a_l = a_cols.long()

    def plain(i):
        probs[i % copies].run(fp6_marlin.mul)

    def fused(**kw):
        def f(i):
            p = probs[i % copies]
            fp6_marlin.mul_fused(p.A, p.B, p.C, p.s, p.ws, p.qc if p.qc else -1, p.gs, **kw)
        return f

    def around(i):                                                      # the same result with separate kernels
        p = probs[i % copies]
        ag = torch.index_select(p.A, 1, a_l)
        fp6_marlin.mul(ag, p.B, p.C, p.s, p.ws, p.qc if p.qc else -1, -1, -1, -1, 16, p.gs)
        torch.index_select(p.C, 1, inv, out=out)
        out.add_(bias).add_(res)

    variants = {"mul": plain, "fused_scatter": fused(c_cols=c_cols), "fused_scatter_layer_map": fused(c_cols=c_layer),
                "fused_gather": fused(a_cols=a_cols),
                "fused_bias_residual": fused(bias=bias, residual=res),
                "fused_all": fused(a_cols=a_cols, c_cols=c_cols, bias=bias, residual=res), "torch_kernels_around_mul": around}
    row = {"fused": f"m={m} {k}x{n} qc={qc} gs={gs}"}
    iters = copies * max(1, 100 // copies)
    for name, f in variants.items():
        for i in range(4):
            f(i)
        torch.cuda.synchronize()
        fn, calls = graphed(torch, f, copies, iters)
        settle(torch, fn, calls)
        _, ev = time_region(torch, fn, calls)
        row[name + "_us"] = round(ev / iters * 1e6, 2)
    print(json.dumps(row), flush=True)


def rows_bench(args):
    """`--rows m,k,n[,quant_rows]`: the row-mixed GEMM (`mul_rows`: INT4 rows and FP6 rows of every column in one
    launch) against what the column-mix entry needs for the same result (one `mul` per row range and an addition),
    both replayed from HIP graphs over rotated weights.  Bytes: INT4 words + FP6 planes + scales, read once."""
    import torch
    import fp6_marlin
    v = [int(x) for x in args.rows.split(",")]
    m, k, n = v[:3]
    qr = v[3] if len(v) > 3 else 256
    k4 = k - qr
    gen = torch.Generator().manual_seed(0)
    fp6_marlin.init(0)
    words4, words6, ns4 = k4 * n // 8, qr * n * 3 // 16, (k4 // 128) * n
    nbytes = 4 * (words4 + words6) + 2 * (ns4 + n)
    copies = max(2, min(24, int(640e6 // nbytes) + 1))
    Bs = [torch.randint(-2 ** 31, 2 ** 31 - 1, (words4 + words6,), generator=gen, dtype=torch.int64).to(torch.int32).cuda()
          for _ in range(copies)]
    ss = [(torch.rand(ns4 + n, generator=gen) * 0.01 + 0.001).half().cuda() for _ in range(copies)]
    parts = [(b[:words4].clone(), b[words4:].clone(), x[:ns4].clone(), x[ns4:].clone()) for b, x in zip(Bs, ss)]
    A = torch.randn((m, k), generator=gen).half().cuda()
    A4, A6 = A[:, :k4].contiguous(), A[:, k4:].contiguous()
    C, C4, C6 = (torch.zeros((m, n), dtype=torch.half, device="cuda") for _ in range(3))
    ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device="cuda")

    def one(i):
        fp6_marlin.mul_rows(A, Bs[i % copies], C, ss[i % copies], ws, qr)

    def two(i):
        b4, b6, s4, s6 = parts[i % copies]
        fp6_marlin.mul(A4, b4, C4, s4, ws, -1, -1, -1, -1, 16, 128)
        fp6_marlin.mul(A6, b6, C6, s6, ws, n, -1, -1, -1, 16, -1)
        torch.add(C4, C6, out=C)

    row = {"rows": f"m={m} {k}x{n} quant_rows={qr}", "weight_bytes": nbytes}
    iters = copies * max(1, 100 // copies)
    for name, f in (("mul_rows", one), ("two_mul_and_add", two)):
        for i in range(4):
            f(i)
        torch.cuda.synchronize()
        fn, calls = graphed(torch, f, copies, iters)
        settle(torch, fn, calls)
        _, ev = time_region(torch, fn, calls)
        row[name + "_us"] = round(ev / iters * 1e6, 2)
    t = row["mul_rows_us"] * 1e-6
    row["weight_GBs"] = round(nbytes / t / 1e9, 1)
    row["hbm_frac"] = round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4)
    row["TFLOPs"] = round(2 * m * k * n / t / 1e12, 2)
    print(json.dumps(row), flush=True)


def pack_bench(args):
    """`--pack k,n[,quant_cols,group_size]`: on-GPU weight preparation (fp16 [k, n] -> B, s) against the host
    packers on the box's cores.  Algorithmic bytes: the fp16 weight read once, the packed words and scales
    written once (no check weight)."""
    import torch
    import fp6_marlin
    v = [int(x) for x in args.pack.split(",")]
    k, n = v[:2]
    qc, gs = (v[2] if len(v) > 2 else 256), (v[3] if len(v) > 3 else 128)
    w = (torch.randn((k, n), generator=torch.Generator().manual_seed(0)) * 0.02).half()
    wd = w.cuda()
    nbytes = 2 * k * n + weight_bytes(k, n, qc, gs)
    for _ in range(2):
        fp6_marlin.pack_mixed_weight_device(wd, qc, gs, True, want_ref=False)
    torch.cuda.synchronize()
    iters = 10
    t0 = time.perf_counter()
    for _ in range(iters):
        fp6_marlin.pack_mixed_weight_device(wd, qc, gs, True, want_ref=False)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / iters
    t0 = time.perf_counter()
    fp6_marlin.pack_mixed_weight(w, qc, gs)
    th = time.perf_counter() - t0
    print(json.dumps({"pack": f"{k}x{n} qc={qc} gs={gs}", "gpu_ms": round(t * 1e3, 3), "gpu_GBs": round(nbytes / t / 1e9, 1),
                      "hbm_frac": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4), "host_ms": round(th * 1e3, 1),
                      "host_threads": os.cpu_count(), "speedup": round(th / t, 1)}), flush=True)


def sweep(args):
    """Per-shape numbers for every benchmark configuration; written as JSON rows."""
    import torch
    import fp6_marlin
    gen = torch.Generator().manual_seed(0)
    fp6_marlin.init(0)
    rows = []
    cases = []
    cases += [("cfg0", 16, 4096, 4096, 256, 128)]
    cases += [("cfg1-7B", 1, k, n, 256, 128) for k, n in LLAMA7B]
    cases += [("cfg1-7B-m16", 16, k, n, 256, 128) for k, n in LLAMA7B]
    cases += [("cfg2-70B", m, k, n, 256, 128) for m in (1, 16) for k, n in LLAMA70B]
    cases += [("cfg3-msweep", m, 8192, 8192, 256, 128) for m in (1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024)]
    cases += [("cfg4-13B", 33, 5120, 13824, 512, -1), ("cfg4-13B", 33, 13824, 5120, 512, -1)]
    cases += [("all-int4-g-1", 16, 8192, 8192, 0, -1), ("all-int4-g128", 16, 8192, 8192, 0, 128)]
    for tag, m, k, n, qc, gs in cases:
        row = measure_shape(torch, fp6_marlin, gen, tag, m, k, n, qc, gs)
        rows.append(row)
        print(json.dumps(row), flush=True)
    os.makedirs(os.path.dirname(os.path.abspath(args.sweep)), exist_ok=True)
    with open(args.sweep, "w") as fh:
        json.dump(rows, fh, indent=1)


def timeline(args):
    """Per-workgroup clock stamps of one GEMM (python fp6-marlin_amd/build.py --timeline builds the instrumented library):
    where the launch's time goes, and how far apart its workgroups end.  Stamps, microseconds after the first workgroup's
    start: decode kernel (one wave per workgroup)  start, first weights landed, loop end, rows formed, atomics issued,
    -, stored / cell cleared, end;  other kernels  start, first weights landed, loop end, slices summed through LDS,
    partial tile published, counted, gathered and stored (last arrival only), end."""
    import ctypes
    import numpy as np
    import torch
    path = os.path.join(ROOT, "fp6-marlin_amd", "fp6_marlin", "libfp6m_timeline.so")
    if not os.path.exists(path):
        sys.exit("bench.py --timeline: build the instrumented library first (python fp6-marlin_amd/build.py --timeline)")
    lib = ctypes.CDLL(path)
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.fp6m_mul.argtypes = [vp] * 4 + [ci] * 3 + [vp, ci, vp] + [ci] * 6
    lib.fp6m_mul.restype = ci
    lib.fp6m_init.argtypes = [ci]
    lib.fp6m_tuning_set.argtypes = [ctypes.c_char_p, ci]
    assert lib.fp6m_init(0) == 0
    vals = [int(x) for x in args.timeline.split(",")]
    m, k, n = vals[:3]
    qc = vals[3] if len(vals) > 3 else 256
    gs = vals[4] if len(vals) > 4 else 128
    for kv in (args.knobs or "").split(","):
        if kv:
            name, value = kv.split("=")
            assert lib.fp6m_tuning_set(name.encode(), int(value)) == 0, f"unknown knob {name}"
    gen = torch.Generator().manual_seed(0)
    copies = max(2, min(8, int(640e6 // weight_bytes(k, n, qc, gs)) + 1))
    probs = [Problem(torch, m, k, n, qc, gs, gen, on_device=True) for _ in range(copies)]
    stamps = torch.zeros(1 << 20, dtype=torch.int64, device="cuda")

    def call(p):
        rc = lib.fp6m_mul(p.A.data_ptr(), p.B.data_ptr(), p.C.data_ptr(), p.s.data_ptr(), p.m, p.n, p.k, p.ws.data_ptr(), 0,
                          torch.cuda.current_stream().cuda_stream, -1, -1, -1, 16, p.qc if p.qc else -1, p.gs)
        assert rc == 0, rc

    t_end = time.perf_counter() + 0.05                     # clocks as in a running loop
    while time.perf_counter() < t_end:
        for p in probs:
            call(p)
    torch.cuda.synchronize()
    os.environ["FP6M_TIMELINE_PTR"] = str(stamps.data_ptr())
    pct = [0, 10, 50, 90, 99, 100]
    reps = []
    for rep in range(16):
        for p in probs[1:]:                                # (other weights in between: nothing of this one is cached)
            call(p)
        stamps.zero_()
        call(probs[0])
        torch.cuda.synchronize()
        t = stamps.cpu().numpy().reshape(-1, 8)
        used = t[:, 0] != 0
        t = t[used].astype(np.float64)
        raw = stamps.cpu().numpy().reshape(-1, 8)[used]
        reps.append(((t - t[:, 0].min()) / 100.0, np.nonzero(used)[0], (raw[:, 5] >> 32) & 15))   # the clock counts 100 MHz
    names = ["start", "first weights", "loop end", "rows / slices summed", "atomics out / published", "counted",
             "stored (last arrival)", "end"]
    out = {"m": m, "k": k, "n": n, "quant_cols": qc, "group_size": gs, "knobs": args.knobs or "", "workgroups": int(len(reps[0][1])),
           "kernel_us": round(float(np.mean([r[0][:, 7].max() for r in reps])), 2), "percentiles": pct, "stamps_us": {}}
    for i, name in enumerate(names):
        if m == 1 and i == 5:
            continue                                       # (the decode kernel keeps its hardware id there)
        rows = [np.percentile(r[0][:, i][r[0][:, i] > 0] if i else r[0][:, i], pct) for r in reps if (r[0][:, i] > 0).any() or i == 0]
        if rows:
            out["stamps_us"][name] = [round(float(v), 2) for v in np.mean(rows, axis=0)]
    # by generation: workgroup index / 8 is the index inside an XCD; the first 4 x CUs / 8 one-wave workgroups of an XCD
    # (CUs / 8 four-wave ones) start on SIMDs (CUs) of their own, the later ones share
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    per_gen = (4 if m == 1 else 1) * cus // 8
    gens = {}
    for r, idx, _ in reps:
        g = (idx >> 3) // per_gen
        for gi in np.unique(g):
            sel = g == gi
            gens.setdefault(int(gi), []).append([sel.sum(), np.median(r[sel, 2]), np.percentile(r[sel, 7], 50), r[sel, 7].max()])
    out["by_generation"] = {str(gi): {"workgroups": int(np.mean([x[0] for x in v])), "loop_end_median_us": round(float(np.mean([x[1] for x in v])), 2),
                                      "end_median_us": round(float(np.mean([x[2] for x in v])), 2),
                                      "end_max_us": round(float(np.mean([x[3] for x in v])), 2)} for gi, v in sorted(gens.items())}
    if m == 1:
        # the decode kernel's waves also note the XCD they run on: the dies do not all stream at the same rate
        xcds = {}
        for r, _, xcc in reps:
            for x in np.unique(xcc):
                xcds.setdefault(int(x), []).append([np.sum(xcc == x), np.median(r[xcc == x, 2]), r[xcc == x, 7].max()])
        out["by_xcd"] = {str(x): {"waves": int(np.mean([v[0] for v in vs])), "loop_end_median_us": round(float(np.mean([v[1] for v in vs])), 2),
                                  "end_max_us": round(float(np.mean([v[2] for v in vs])), 2)} for x, vs in sorted(xcds.items())}
    print(json.dumps(out), flush=True)


def regret(args):
    """The planners against forced plans: for each shape the default call and every forced (waves per workgroup, k parts)
    plan of the kernel that serves that row count (m = 1: forced uniform chunk lengths), all replayed from HIP graphs over
    rotated weights; `regret` = default time / best forced time - 1.  --regret KIND[,GROUP_SIZE] with KIND decode (m = 1),
    m16 (m = 6 and 16) or mb (m = 32, 64, 128); the shapes are k = 2048 .. 11008 x 20 .. 172 column tiles unless --shape
    names one.  This is how the dispatcher's rules were fitted; on another chip it shows where they no longer hold."""
    import torch
    import fp6_marlin
    from fp6_marlin import cabi
    kind, _, gs_text = args.regret.partition(",")
    gs = int(gs_text) if gs_text else 128
    assert kind in ("decode", "m16", "mb"), "--regret decode|m16|mb[,group_size]"
    fp6_marlin.init(0)
    gen = torch.Generator().manual_seed(0)
    rows = {"decode": [1], "m16": [6, 16], "mb": [32, 64, 128]}[kind]
    if args.shape:
        m, k, n = [int(x) for x in args.shape.split(",")[:3]]
        shapes = [(m, k, n)]
    else:
        shapes = [(m, k, t * 128) for m in rows for k in (2048, 3072, 4096, 5120, 8192, 11008)
                  for t in (20, 32, 44, 60, 72, 88, 104, 120, 172)]
    parts = (1, 2, 3, 4, 5, 6, 8, 10, 12, 16)

    def plans(m, k):
        if kind == "decode":
            units = k // (128 if gs == 128 else 64)
            return [{"share": q} for q in parts if q <= units]
        if kind == "m16":
            return [{"wk16": wk, "ksplit": c} for wk in (4, 8) for c in parts if c <= 8 and k // (32 * wk * c) >= 2]
        blocks = [2, 4] if m <= 32 else ([4] if m <= 64 else [4, 8])
        return [{"mb": b, "wk": wk, "ksplit": c} for b in blocks for wk in ((4, 8) if b != 8 else (4,)) for c in parts
                if c <= 8 and k // (32 * wk * c) >= 2]

    def knobs(plan):
        cabi.lib.fp6m_tuning_set(None, 0)
        for name, value in plan.items():
            assert cabi.lib.fp6m_tuning_set(name.encode(), int(value)) == 0, name

    worst, total, count = 0.0, 0.0, 0
    for m, k, n in shapes:
        qc = 256
        copies = max(2, min(24, int(640e6 // weight_bytes(k, n, qc, gs)) + 1))
        probs = [Problem(torch, m, k, n, qc, gs, gen, on_device=True) for _ in range(copies)]
        iters = copies * max(1, 48 // copies)
        fns = []
        for plan in [{}] + plans(m, k):
            knobs(plan)
            try:
                probs[0].run(fp6_marlin.mul)
                torch.cuda.synchronize()
                fns.append((plan,) + graphed(torch, lambda i: probs[i % copies].run(fp6_marlin.mul), copies, iters))
            except RuntimeError:                                         # (a forced plan the scratch cannot hold)
                torch.cuda.synchronize()
        cabi.lib.fp6m_tuning_set(None, 0)
        times = {}
        for _ in range(2):
            for plan, fn, calls in fns:
                settle(torch, fn, calls, ms=15)
                _, ev = time_region(torch, fn, calls)
                key = json.dumps(plan, sort_keys=True)
                times[key] = min(times.get(key, 1e9), ev / iters * 1e6)
        default = times.pop("{}")
        best = min(times, key=times.get)
        r = default / times[best] - 1.0
        worst, total, count = max(worst, r), total + max(r, 0.0), count + 1
        print(json.dumps({"m": m, "k": k, "n": n, "group_size": gs, "default_us": round(default, 2), "best_forced_us": round(times[best], 2),
                          "best_forced": json.loads(best), "regret": round(r, 4)}), flush=True)
        del probs, fns
        torch.cuda.empty_cache()
    print(json.dumps({"kind": kind, "group_size": gs, "shapes": count, "mean_regret": round(total / count, 4), "worst_regret": round(worst, 4)}),
          flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--sweep", type=str, default=None, help="write the per-shape table of all configs to this file")
    ap.add_argument("--shape", type=str, default=None, help="m,k,n[,quant_cols,group_size]: measure one shape")
    ap.add_argument("--layout", type=str, default="reference", choices=["reference", "gfx950"],
                    help="word order of the packed weight for --shape (gfx950: after repack_gfx950)")
    ap.add_argument("--fused", type=str, default=None, help="m,k,n[,quant_cols,group_size]: time mul_fused against mul + torch kernels")
    ap.add_argument("--rows", type=str, default=None, help="m,k,n[,quant_rows]: time the row-mixed GEMM against two mul calls and an addition")
    ap.add_argument("--pack", type=str, default=None, help="k,n[,quant_cols,group_size]: time the on-GPU weight packer")
    ap.add_argument("--models", action="store_true", help="the reference's own benchmark: its five models' layers at batch 16, "
                                                          "quant_cols -1 and 256, per-channel scales, time-weighted speed-up over fp16")
    ap.add_argument("--headline-only", action="store_true", help="skip the other regimes' rows of the JSON line")
    ap.add_argument("--no-graph", action="store_true", help="launch every GEMM from Python instead of replaying a HIP graph")
    ap.add_argument("--timeline", type=str, default=None, help="m,k,n[,quant_cols,group_size]: per-workgroup clock stamps of one GEMM "
                    "(needs fp6-marlin_amd/build.py --timeline)")
    ap.add_argument("--knobs", type=str, default=None, help="with --timeline: tuning knobs, name=value[,name=value]")
    ap.add_argument("--regret", type=str, default=None, help="decode|m16|mb[,group_size]: the default plan against every forced plan "
                    "(with --shape m,k,n: that shape only)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="for `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE`: one 256 MiB device copy, then one layer of GEMMs")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the op shards along N without any exchange); "
                 "run with --gpus 1")
    if args.traffic_probe:
        traffic_probe()
    elif args.regret:
        regret(args)
    elif args.timeline:
        timeline(args)
    elif args.models:
        import torch
        import fp6_marlin
        fp6_marlin.init(0)
        for row in reference_models(torch, fp6_marlin, torch.Generator().manual_seed(0)):
            print(json.dumps(row), flush=True)
    elif args.sweep:
        sweep(args)
    elif args.shape:
        one_shape(args)
    elif args.pack:
        pack_bench(args)
    elif args.fused:
        fused_bench(args)
    elif args.rows:
        rows_bench(args)
    else:
        headline(args)


if __name__ == "__main__":
    main()
