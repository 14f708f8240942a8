#!/usr/bin/env python3
"""MoE-layer throughput of the W8A8 fused-MoE path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--tokens M]

Without --workload the line's headline is the DeepSeek-V3-shape W8A8 decode layer (128 tokens,
shared expert included) with its CPU baseline, and the other benchmark configurations (prefill,
the Qwen3 shape, the fp8 layers) are timed in the same run and reported under "workloads".

A step is one call of the whole layer (routing -> align -> int8 quant -> gate_up
GEMM + SiLU-mul -> int8 quant -> down GEMM -> combine, plus the shared expert
where the shape has one) over one batch of synthetic tokens that already sits
in HBM. Prints ONE JSON line: tokens/s, the roofline of the dominant kernel
(HIP events recorded around it inside the timed calls) and the CPU baseline
(the torch-CPU restatement of the reference's expert loop, timed on this host).
"""
import argparse
import ctypes as C
import json
import math
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "vllm-kunlun_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E

WORKLOAD_LABEL = {
    "qwen3-decode": "Qwen3-MoE-30B-A3B-shape MoE layer, W8A8 int8, decode, 64 tokens",
    "qwen3-prefill": "Qwen3-MoE-30B-A3B-shape MoE layer, W8A8 int8, prefill, 8192 tokens",
    "qwen3-prefill-skew": "Qwen3-MoE-30B-A3B-shape MoE layer, W8A8 int8, prefill, 8192 tokens, +2.0 logit bias on 8 experts",
    "dsv3-decode": "DeepSeek-V3-shape MoE layer (+1 shared expert), W8A8 int8, decode, 128 tokens",
    "dsv3-prefill": "DeepSeek-V3-shape MoE layer (+1 shared expert), W8A8 int8, prefill, 4096 tokens",
    "kimi-decode": "Kimi-K2-shape MoE layer (384 experts, +1 shared), W8A8 int8, decode, 128 tokens",
    "kimi-prefill": "Kimi-K2-shape MoE layer (384 experts, +1 shared), W8A8 int8, prefill, 4096 tokens",
    "dsv3-fp8-decode": "DeepSeek-V3-shape MoE layer (+1 shared expert), fp8-e4m3 128x128-block weights, decode, 128 tokens",
    "dsv3-fp8-prefill": "DeepSeek-V3-shape MoE layer (+1 shared expert), fp8-e4m3 128x128-block weights, prefill, 4096 tokens",
    "kimi-fp8-decode": "Kimi-K2-shape MoE layer (384 experts, +1 shared), fp8-e4m3 128x128-block weights, decode, 128 tokens",
    "kimi-fp8-prefill": "Kimi-K2-shape MoE layer (384 experts, +1 shared), fp8-e4m3 128x128-block weights, prefill, 4096 tokens",
    "qwen3-bf16-decode": "Qwen3-MoE-30B-A3B-shape MoE layer, bf16 weights (no quantization), decode, 64 tokens",
    "qwen3-bf16-prefill": "Qwen3-MoE-30B-A3B-shape MoE layer, bf16 weights (no quantization), prefill, 8192 tokens",
    "qwen3-w4a16-decode": "Qwen3-MoE-30B-A3B-shape MoE layer, 4-bit weights (groups of 128) and bf16 activations, "
                          "decode, 64 tokens",
    "qwen3-w4a16-prefill": "Qwen3-MoE-30B-A3B-shape MoE layer, 4-bit weights (groups of 128) and bf16 activations, "
                           "prefill, 8192 tokens",
    "kimi-w4a16-decode": "Kimi-K2-shape MoE layer (384 experts, no shared expert), 4-bit weights (groups of 32) and bf16 "
                         "activations, decode, 128 tokens",
    "kimi-w4a16-prefill": "Kimi-K2-shape MoE layer (384 experts, no shared expert), 4-bit weights (groups of 32) and bf16 "
                          "activations, prefill, 4096 tokens",
    "tiny-bf16": "tiny bf16 MoE layer (32 tokens, hidden 512, 8 experts, top-2, intermediate 256), no quantization",
}
PEAK_TOPS = {"int8": 5000.0, "fp8": 5000.0, "none": 2500.0, "w4": 2500.0}  # MI355X dense MFMA: int8, fp8, bf16
DTYPE = {"int8": "int8", "fp8": "fp8_e4m3", "none": "bf16", "w4": "bf16 (4-bit weights)"}


class HipEvents:
    """hipEvent_t handles made through the HIP runtime torch already loaded."""

    def __init__(self, n):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [C.c_void_p]
        self.hip.hipEventDestroy.argtypes = [C.c_void_p]
        self.handles = (C.c_void_p * n)()
        for i in range(n):
            ev = C.c_void_p()
            rc = self.hip.hipEventCreate(C.byref(ev))
            assert rc == 0, f"hipEventCreate failed: {rc}"
            self.handles[i] = ev

    def elapsed_ms(self, i, j):
        self.hip.hipEventSynchronize(self.handles[j])
        ms = C.c_float()
        rc = self.hip.hipEventElapsedTime(C.byref(ms), self.handles[i], self.handles[j])
        assert rc == 0, f"hipEventElapsedTime failed: {rc}"
        return ms.value

    def close(self):
        for h in self.handles:
            self.hip.hipEventDestroy(h)


def algorithmic_work(shape, n_active):
    """Bytes that must cross HBM and int8 operations that must run, per layer call
    and for each GEMM launch, from the shape and the number of experts hit."""
    M, H, E, K, I, Is, P = shape.M, shape.H, shape.E, shape.K, shape.I, shape.I_shared, shape.P
    wb = {"none": 2, "w4": 0.5}.get(shape.quant, 1)  # bytes per weight
    ab = 2 if shape.quant in ("none", "w4") else 1    # bytes per activation value / code

    def w_bytes(n, k):  # one [n,k] weight matrix with its scales
        return int(n * k * wb) + {"int8": n * 4, "fp8": (n // 128) * (k // 128) * 4, "none": 0,
                                  "w4": n * (k // shape.group_size) * 2}[shape.quant]

    def a_bytes(rows, k):  # (quantised) activations of `rows` rows with their scales
        return rows * k * ab + {"int8": rows * 4, "fp8": rows * (k // 128) * 4, "none": 0, "w4": 0}[shape.quant]

    g1_bytes = n_active * w_bytes(2 * I, H) + a_bytes(M, H) + P * 4 + P * I * 2
    g2_bytes = n_active * w_bytes(H, I) + a_bytes(P, I) + P * H * 2
    shared_bytes = (w_bytes(2 * Is, H) + w_bytes(H, Is)) if Is else 0
    if Is == I and shape.quant == "int8":  # the shared expert runs inside the two routed GEMM launches
        g1_bytes += w_bytes(2 * Is, H) + M * Is * 2
        g2_bytes += w_bytes(H, Is) + a_bytes(M, Is) + M * H * 2
    layer_bytes = (n_active * (w_bytes(2 * I, H) + w_bytes(H, I)) + shared_bytes + 2 * M * H * 2 + M * E * 4)
    fold = M if (Is == I and shape.quant == "int8") else 0
    g1_ops = 2 * (P + fold) * 2 * I * H
    g2_ops = 2 * (P + fold) * H * I
    layer_ops = g1_ops + g2_ops + 2 * M * 3 * Is * H
    return dict(g1_bytes=g1_bytes, g2_bytes=g2_bytes, layer_bytes=layer_bytes, g1_ops=g1_ops, g2_ops=g2_ops,
                layer_ops=layer_ops)


def measured_traffic(workload):
    """HBM bytes per launch of the gate_up GEMM from the committed counter summary
    (profiles/<workload>_gemm1_traffic.txt, line 'traffic_bytes_per_launch = N'), or None."""
    path = os.path.join(ROOT, "profiles", f"{workload}_gemm1_traffic.txt")
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch"):
                    return float(line.split("=")[1])
    except OSError:
        pass
    return None


def cpu_baseline(sl, budget_s=15.0):
    """The reference's torch expert loop (oracle/torch_moe.py) on the host cores: one warm-up
    call, then whole layer calls of the same workload for about budget_s seconds."""
    import torch
    from oracle import torch_moe as tm
    s = sl.shape
    host = lambda t: None if t is None else t.detach().cpu()  # noqa: E731
    w13, w13_max, w2, w2_max, shared = sl.host_weights()  # row-major copies of the (tiled) device weights
    if s.quant == "int8":
        fn, what = tm.w8a8_moe, "torch-CPU restatement of the reference expert loop"
        args = (host(sl.x), host(sl.logits), w13, w13_max, w2, w2_max, s.K, s.scoring, True, s.n_group, s.topk_group,
                s.routed_scale, host(sl.bias), shared)
    elif s.quant == "none":
        fn, what = tm.bf16_moe, "torch-CPU restatement of the reference expert loop"
        args = (host(sl.x), host(sl.logits), w13, w2, s.K, True)
    else:
        return None  # no CPU restatement of the fp8 / 4-bit layers is timed
    t0 = time.perf_counter()
    fn(*args)  # warm-up
    first = time.perf_counter() - t0
    runs = max(1, min(600, int(budget_s / max(first, 1e-3))))  # about budget_s seconds of CPU work
    times = []
    for _ in range(runs):
        t0 = time.perf_counter()
        fn(*args)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": s.M / med, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{runs} full layer call(s) of the same workload ({s.M} tokens) after 1 warm-up, median; "
                      f"{what}; host has {os.cpu_count()} cpus"}


def vendor_dense_gemm(shape, g1_ops, peak_tops, reps=20):
    """The vendor library's dense GEMM of the gate_up GEMM's size, as a yardstick only: one
    [H,2I] weight matrix for all P rows (no experts, no gather, no dequantisation, no SiLU-mul)."""
    import torch
    P, H, N = shape.P, shape.H, 2 * shape.I
    if shape.quant == "int8":
        x = torch.randint(-127, 128, (P, H), dtype=torch.int8, device="cuda:0")
        w = torch.randint(-127, 128, (N, H), dtype=torch.int8, device="cuda:0")
        fn, what = (lambda: torch._int_mm(x, w.t())), "torch._int_mm (int8 x int8 -> int32)"
    else:
        x = torch.randn(P, H, device="cuda:0").bfloat16()
        w = torch.randn(N, H, device="cuda:0").bfloat16()
        fn, what = (lambda: x @ w.t()), "torch bf16 matmul"
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / reps
    ops = 2.0 * P * H * N
    return {"what": f"{what}, [{P},{H}] x [{H},{N}]", "ms": ms, "tops": ops / ms / 1e9,
            "frac_of_peak": ops / ms / 1e9 / peak_tops}


# What plain `python bench.py` runs besides the headline workload: the other benchmark
# configurations, reported under "workloads" in the same JSON line.
SUITE = ["dsv3-prefill", "qwen3-decode", "qwen3-prefill", "qwen3-prefill-skew", "dsv3-fp8-decode", "dsv3-fp8-prefill",
         "kimi-decode", "kimi-prefill", "kimi-fp8-decode", "kimi-fp8-prefill"]
HEADLINE = "dsv3-decode"


def clock_probe(plan, stream, ms_per_step, load_ms=20.0):
    """Shader clock beside the layer: kmoe_clock_probe runs on a second stream (the library leaves CUs free for
    it: KMOE_SPARE_CUS, set by main) while the layer is called back to back for about load_ms. Returns the clock
    by the probe's s_sleep runs (s_memtime ticks / duration by the 100 MHz counter) before the load and during
    it, and the ticks of its fixed v_fma chain in both phases (equal ticks = s_memtime follows the shader clock)."""
    import numpy as np
    import torch
    from vllm_kunlun_amd import _lib as L
    n_wg, reps = 16, 4096
    samples = torch.zeros(n_wg * reps * 3, dtype=torch.int64, device="cuda:0")
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    t_probe = time.perf_counter()
    L.check(L.lib.kmoe_clock_probe(L.ptr(samples), n_wg, reps, side.cuda_stream))
    time.sleep(0.004)
    t_load0 = time.perf_counter() - t_probe
    with torch.cuda.stream(stream):
        for _ in range(max(3, int(load_ms / ms_per_step))):
            plan()
        stream.synchronize()
    t_load1 = time.perf_counter() - t_probe
    torch.cuda.synchronize()
    r = samples.cpu().numpy().reshape(n_wg, reps, 3).astype(np.float64)
    t = (r[:, :, 0] - r[:, :, 0].min()) * 1e-8          # seconds since the first sample
    ghz = r[:, :, 2] / (r[:, :, 1] * 10.0)               # ticks per ns
    sleep, fma = np.zeros(reps, bool), np.zeros(reps, bool)
    sleep[1::2], fma[0::2] = True, True
    # host and device clocks both run in real time: the load's window, a millisecond inside its host-side bounds
    idle = t < (t_load0 - 1e-3)
    busy = (t > t_load0 + 1.5e-3) & (t < t_load1 - 1.0e-3)

    def med(mask, col):
        v = col[mask]
        return float(np.median(v)) if v.size else None
    return {
        "probe": f"{n_wg} single-wave workgroups beside the layer, {reps} runs each; the tile kernels leave "
                 f"{os.environ.get('KMOE_SPARE_CUS', '0')} CUs free",
        "idle_ghz": med(idle & sleep[None, :], ghz), "loaded_ghz": med(busy & sleep[None, :], ghz),
        "loaded_ghz_p10_p90": [float(x) for x in np.percentile(ghz[busy & sleep[None, :]], [10, 90])] if busy.any() else None,
        "sleep_run_ticks_idle": med(idle & sleep[None, :], r[:, :, 2]), "sleep_run_ticks_loaded": med(busy & sleep[None, :], r[:, :, 2]),
        "sleep_run_ns_idle": med(idle & sleep[None, :], r[:, :, 1] * 10.0), "sleep_run_ns_loaded": med(busy & sleep[None, :], r[:, :, 1] * 10.0),
        "fma_chain_ticks_idle": med(idle & fma[None, :], r[:, :, 2]), "fma_chain_ticks_loaded": med(busy & fma[None, :], r[:, :, 2]),
        "fma_chain_ns_idle": med(idle & fma[None, :], r[:, :, 1] * 10.0), "fma_chain_ns_loaded": med(busy & fma[None, :], r[:, :, 1] * 10.0),
        "samples_idle": int((idle & sleep[None, :]).sum()), "samples_loaded": int((busy & sleep[None, :]).sum()),
    }


def measure(a, workload, shape, label, sl, with_cpu_baseline, exact_steps=True):
    """Times one workload's layer on cuda:0 (inputs resident in HBM) and returns the pieces of
    the JSON line: ms per step (graph replay / eager plan / plugin entry), per-stage durations
    from HIP events on the launch stream, the gate_up GEMM's roofline, the layer's fractions."""
    import torch
    from vllm_kunlun_amd import _lib as L
    from vllm_kunlun_amd._plan import make_moe_plan

    lay = sl.layer
    x, logits = sl.x.contiguous(), sl.logits.contiguous()
    out = torch.empty_like(x)
    fmt = {"int8": L.KMOE_FMT_INT8, "fp8": L.KMOE_FMT_FP8_BLOCK, "none": L.KMOE_FMT_BF16,
           "w4": L.KMOE_FMT_W4A16}[shape.quant]
    w4 = shape.quant == "w4"

    w_gate = None
    if a.router:
        gen = torch.Generator(device="cuda:0")
        gen.manual_seed(a.seed + 1)
        w_gate = (torch.randn(shape.E, shape.H, generator=gen, device="cuda:0") * shape.H ** -0.5).to(x.dtype)  # logits ~ N(0,1)

    def make_plan(stage_events=None):
        # the argument block the plugin methods build (apply_monolithic / KunlunOps.fused_moe)
        return make_moe_plan(fmt, x, None if a.router else logits, out, shape.K,
                             lay.w13_weight_packed if w4 else lay.w13_weight,
                             lay.w2_weight_packed if w4 else lay.w2_weight,
                             getattr(lay, "w13_weight_scale", None), getattr(lay, "w2_weight_scale", None),
                             shape.scoring, True, shape.n_group, shape.topk_group, shape.routed_scale, sl.bias,
                             sl.shared, 1.0, stage_events, router_weight=w_gate,
                             group_size=shape.group_size if w4 else None, tile_variant=a.tile_variant,
                             side_stream=not a.one_stream)

    # The layer, its inputs and the workspace were produced on the default stream;
    # finish that work before a second stream touches (recycled) memory.
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        plan = make_plan()
        if a.copy_probe:
            src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0")
            torch.bitwise_not(src, out=torch.empty_like(src))
        for _ in range(3):
            plan()
        # which GEMM kernels the launchers chose for this call, as the library itself reports them
        L.lib.kmoe_trace_kernels(1)
        plan()
        L.lib.kmoe_trace_kernels(0)
        traced = L.lib.kmoe_traced_kernels().decode().splitlines()
        stream.synchronize()

        # The headline workload times exactly --steps steps. The other workloads of the suite time at least
        # kMinTimedMs of work: 20 steps of a 0.1 ms layer are 2 ms between two synchronisations, whose own
        # cost (the first launch after an idle stream, the wake-up at the end) then reads as 4-6 % of a step.
        kMinTimedMs = 20.0
        steps_used = [a.steps]

        def timed(step):
            n = a.steps
            while True:
                for _ in range(a.warmup):
                    step()
                stream.synchronize()
                t0 = time.perf_counter()
                for _ in range(n):
                    step()
                stream.synchronize()
                total = (time.perf_counter() - t0) * 1e3
                if exact_steps or total >= kMinTimedMs or n >= 4000:
                    steps_used[0] = max(steps_used[0], n)
                    return total / n
                n = min(4000, max(n + 1, int(math.ceil(n * kMinTimedMs / total * 1.1))))

        launch_ms = {}
        if a.launch in ("auto", "graph"):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                plan()
            launch_ms["hipgraph replay"] = timed(graph.replay)
        if a.launch in ("auto", "eager"):
            launch_ms["eager"] = timed(plan)
        launch_mode = min(launch_ms, key=launch_ms.get)
        ms_per_step = launch_ms[launch_mode]
        # the plugin entry itself (per-call output allocation, argument block, workspace lookup):
        # reported beside the replayed argument block, never as `value`
        if not a.router and not w4:
            method = lay.quant_method
            kw = sl.apply_kwargs() if shape.quant in ("int8", "fp8") else {}
            launch_ms["apply_monolithic eager"] = timed(lambda: method.apply_monolithic(lay, x, logits, **kw))

        probe = clock_probe(plan, stream, ms_per_step) if a.clock_probe else None

        # the same calls again with HIP events around each stage (eager: events are
        # not captured), for the per-kernel durations of the roofline
        ev = HipEvents(2 * len(L.STAGES))
        plan_ev = make_plan(ev.handles)
        stage_ms = {s: 0.0 for s in L.STAGES}
        for it in range(a.warmup + a.steps):
            plan_ev()
            if it >= a.warmup:
                for i, s in enumerate(L.STAGES):
                    stage_ms[s] += ev.elapsed_ms(2 * i, 2 * i + 1)
        stage_ms = {s: v / a.steps for s, v in stage_ms.items()}
        stream.synchronize()
        ev.close()
    torch.cuda.current_stream().wait_stream(stream)

    lod = plan.view("lod", shape.E + 1, torch.int32).cpu()
    n_active = int(((lod[1:] - lod[:-1]) > 0).sum())
    work = algorithmic_work(shape, n_active)
    intensity = work["layer_ops"] / work["layer_bytes"]
    peak_tops = PEAK_TOPS[shape.quant]
    hbm_bound = intensity < peak_tops * 1e12 / (HBM_PEAK_GBS * 1e9)
    g1_s = stage_ms["gemm1"] * 1e-3
    # the launch(es) noted under the first "[gate_up, ...]" heading (two when the device decides between tile shapes)
    heads = [i for i, line in enumerate(traced) if line.startswith("[")] + [len(traced)]
    first = next((n for n, i in enumerate(heads[:-1]) if traced[i].startswith("[gate_up, routed")), None)
    g1_kernel = " | ".join(traced[heads[first] + 1: heads[first + 1]]) if first is not None else "?"
    traffic = None if (a.tokens or a.dims) else measured_traffic(workload)  # the counter summaries are of the named workload
    if hbm_bound:
        achieved = work["g1_bytes"] / g1_s / 1e9
        roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": achieved / HBM_PEAK_GBS, "traffic": traffic}
    else:
        achieved = work["g1_ops"] / g1_s / 1e12
        roofline = {"bound": "mfma", "achieved": achieved, "peak": peak_tops,
                    "unit": "TOP/s" if shape.quant == "int8" else "TFLOP/s",
                    "frac": achieved / peak_tops, "traffic": traffic}
    roofline.update(kernel=g1_kernel + " (gate_up + SiLU-mul)", kernel_ms=stage_ms["gemm1"],
                    algorithmic_bytes=work["g1_bytes"], algorithmic_ops=work["g1_ops"],
                    hbm_frac=work["g1_bytes"] / g1_s / 1e9 / HBM_PEAK_GBS,
                    mfma_frac=work["g1_ops"] / g1_s / 1e12 / peak_tops)

    t_s = ms_per_step * 1e-3
    res = {
        "value": shape.M / t_s,
        "ms_per_step": ms_per_step,
        "dtype": DTYPE[shape.quant].replace("bf16", "f16") if a.act_dtype == "f16" else DTYPE[shape.quant],
        "config": {"workload": label, "name": workload, "tokens": shape.M, "hidden": shape.H,
                   "experts": shape.E, "top_k": shape.K, "moe_intermediate": shape.I,
                   "shared_intermediate": shape.I_shared, "routing": shape.scoring, "experts_hit": n_active,
                   "launch": launch_mode, "launch_ms_per_step": launch_ms, "timed_steps": steps_used[0], "seed": a.seed,
                   "side_stream": not a.one_stream, "router_gemm_inside": bool(a.router), "tile_variant": a.tile_variant, "gemm_kernels": traced,
                   "activations": "float16" if a.act_dtype == "f16" else "bfloat16"},
        "roofline": roofline,
        "layer": {"hbm_gbs": work["layer_bytes"] / t_s / 1e9, "hbm_frac": work["layer_bytes"] / t_s / 1e9 / HBM_PEAK_GBS,
                  "tops": work["layer_ops"] / t_s / 1e12,
                  "mfma_frac": work["layer_ops"] / t_s / 1e12 / peak_tops,
                  "algorithmic_bytes": work["layer_bytes"], "algorithmic_ops": work["layer_ops"],
                  "stage_ms": stage_ms,
                  # what a stage with no launch in it reads (two event records back to back): every entry of
                  # stage_ms carries about this much on top of its kernels, so their sum exceeds ms_per_step
                  "stage_event_overhead_ms": min(stage_ms.values())},
    }
    if a.yardstick and shape.quant in ("int8", "none"):
        res["vendor_dense_gemm"] = vendor_dense_gemm(shape, work["g1_ops"], peak_tops)
    if probe is not None:
        res["clock_probe"] = probe
    res["cpu_baseline"] = cpu_baseline(sl, a.cpu_budget) if with_cpu_baseline else None
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOAD_LABEL),
                    help=f"time this workload alone. Default: {HEADLINE} as the line's headline, with its CPU "
                         f"baseline, and the other configurations ({', '.join(SUITE)}) under 'workloads'")
    ap.add_argument("--no-suite", action="store_true", help="with the default headline: leave out 'workloads'")
    ap.add_argument("--launch", default="auto", choices=["auto", "graph", "eager"],
                    help="replay the layer from a captured HIP graph (as a serving engine does), launch it eagerly, "
                         "or (auto) time K steps each way and report the faster; config.launch says which")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-budget", type=float, default=15.0, help="seconds of CPU work for the baseline sample")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--act-dtype", default="bf16", choices=["bf16", "f16"],
                    help="16-bit type of the activations (and of unquantized weights / 4-bit group scales): the layer "
                         "computes in the same arithmetic type either way")
    ap.add_argument("--tokens", type=int, default=0,
                    help="run the workload's layer at another batch (tokens per call); the config then says so")
    ap.add_argument("--router", action="store_true",
                    help="hand the layer the bf16 gate weight [E,H] instead of router logits: the router GEMM "
                         "then runs inside each step (reported in config; not the default workload)")
    ap.add_argument("--dims", default="",
                    help="other layer dimensions for the workload's format and routing, e.g. "
                         "H=4096,E=8,K=2,I=14336,I_shared=0 (Mixtral-8x7B), or a skewed routing, hot_experts=32,hot_bias=1.0 "
                         "(that bias on the logits of 32 experts); the config then says so")
    ap.add_argument("--tile-variant", type=int, default=0,
                    help="tuning variant of the int8 / fp8 tile kernel for the routed GEMMs of prefill-sized batches "
                         "(kmoe_moe_args.tile_variant; 12: sibling m-tiles paced so that they share weight bytes in L2, "
                         "14: one 8-wave tile of 192 rows per workgroup)")
    ap.add_argument("--one-stream", action="store_true",
                    help="keep every launch on the one stream (the C ABI's default). Without it the layer is called with "
                         "KMOE_FLAG_SIDE_STREAM: a shared expert that cannot ride in the routed launches (the fp8 layers at "
                         "decode sizes) runs on the library's second stream beside them; config.side_stream says which")
    ap.add_argument("--yardstick", action="store_true",
                    help="also time the vendor library's dense GEMM (torch._int_mm / bf16 matmul) with the gate_up "
                         "GEMM's operation count: [P,H] x [H,2I], one weight matrix, no gather, no epilogue")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one bitwise_not over 256 MiB (a kernel of known HBM traffic and a name nothing "
                         "else here has) before the timed region: the yardstick for FETCH_SIZE / WRITE_SIZE runs")
    ap.add_argument("--clock-probe", action="store_true",
                    help="also run the library's shader-clock probe on a second stream beside the layer and report the "
                         "clock it sees idle and under the layer ('clock_probe'); sets KMOE_SPARE_CUS=16 so that the "
                         "persistent tile kernels leave the probe 16 CUs (the layer is a few percent slower for it)")
    ap.add_argument("--zero-operands", action="store_true",
                    help="a power experiment: activations and expert weights all zero (same routing, same kernels, same "
                         "instruction stream, no bit toggles in the data paths); 'data' then says so")
    a = ap.parse_args()
    if a.clock_probe:
        os.environ["KMOE_SPARE_CUS"] = "16"  # read by the library at its first tile launch
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build measures ONE GPU; the layer does not span GPUs (run with --gpus 1)")

    import torch
    from vllm_kunlun_amd import synth

    torch.cuda.set_device(0)
    headline = a.workload or HEADLINE
    names = [headline] + ([] if (a.workload or a.no_suite or a.tokens or a.dims or a.router) else SUITE)

    def shape_of(name):
        shape, label = synth.SHAPES[name], WORKLOAD_LABEL[name]
        if a.tokens and a.tokens != shape.M:
            shape = synth.scaled(shape, M=a.tokens)
            label = re.sub(r"(decode|prefill), \d+ tokens", f"{a.tokens} tokens (batch set by --tokens)", label)
        if a.dims:
            allowed = {"H": int, "E": int, "K": int, "I": int, "I_shared": int, "n_group": int, "topk_group": int,
                       "scoring": str, "routed_scale": float, "hot_experts": int, "hot_bias": float}
            over = {}
            for item in a.dims.split(","):
                key, _, val = item.partition("=")
                if key not in allowed:
                    sys.exit(f"bench.py: --dims takes {sorted(allowed)}, not {key!r}")
                over[key] = allowed[key](val)
            shape = synth.scaled(shape, **over)
            label = f"MoE layer with --dims {a.dims} on the format and routing of {name}, {shape.M} tokens"
        return shape, label

    # workloads that differ only in the batch (tokens, logit bias) share one set of weights:
    # the 11 GB layers are generated once
    def weights_key(s):
        return (s.H, s.E, s.K, s.I, s.scoring, s.n_group, s.topk_group, s.routed_scale, s.I_shared, s.quant,
                s.group_size)

    results, cached = {}, None
    order = sorted(names, key=lambda n: (n != headline,))  # headline first (stable for the rest)
    for name in order:
        shape, label = shape_of(name)
        if cached is not None and cached[0] == weights_key(shape):
            sl = synth.rebatch(cached[1], shape, seed=a.seed)
        else:
            cached = None
            torch.cuda.empty_cache()
            sl = synth.make_layer(shape, "cuda:0", seed=a.seed,
                                  dtype=torch.float16 if a.act_dtype == "f16" else torch.bfloat16)
        cached = (weights_key(shape), sl)
        if a.zero_operands:
            sl.x.zero_()
            for t in (getattr(sl.layer, n, None) for n in ("w13_weight", "w2_weight", "w13_weight_packed", "w2_weight_packed")):
                if t is not None:
                    t.data.zero_()
        results[name] = measure(a, name, shape, label, sl, name == headline and not a.no_cpu_baseline,
                                exact_steps=name == headline)
        print(f"bench.py: {name}: {results[name]['ms_per_step']:.4f} ms/step", file=sys.stderr, flush=True)

    head = results[headline]
    result = {
        "metric": "MoE-layer tokens/s at 1 GPU",
        "value": head["value"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic, all-zero activations and expert weights (--zero-operands)" if a.zero_operands else "synthetic",
        "config": head["config"],
        "roofline": head["roofline"],
        "layer": head["layer"],
        "cpu_baseline": head["cpu_baseline"],
    }
    for extra in ("vendor_dense_gemm", "clock_probe"):
        if extra in head:
            result[extra] = head[extra]
    if len(results) > 1:
        result["workloads"] = {
            n: {"tokens_per_s": r["value"], "ms_per_step": r["ms_per_step"], "dtype": r["dtype"], "config": r["config"],
                "roofline": r["roofline"], "layer": r["layer"]}
            for n, r in results.items() if n != headline}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
